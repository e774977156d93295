"""rocprofv3 profile of one bench.py workload: kernel trace, HBM traffic, shader counters.

    python profile_step.py --workload gdn-int8-g128 [--out profiles] [--sets trace,hbm,shader]

Runs ``bench.py --workload W --no-cpu-baseline`` under rocprofv3, once per pass, from /tmp with TMPDIR=/tmp: the
kernel trace with bench.py's own step counts (the command of the bench line, so the two averages can be compared),
then one run per counter set (the profiler does not split counters over passes) with ``--steps 16 --warmup 16`` (two
fold periods of m = 8 after two of warm-up; counter collection serialises the launches), and the same passes over
``bench.py --calibrate-copy`` for the two HBM counters (a device copy of known size: what FETCH_SIZE / WRITE_SIZE read
for it gives the factor their readings are scaled by).  Writes

    <out>/<workload>_step_kernel.txt    the summary (commands, per-step-of-period durations, counters per dispatch)
    <out>/hbm_traffic.json              {workload: {"traffic": bytes per launch averaged over a fold period, ...}}

``bench.py`` reads the second file for ``roofline.traffic``.  Nothing here touches the GPU itself; every profiled
program is a child process started as ``rocprofv3 ... -- python3 bench.py ...``.
"""
import argparse
import collections
import csv
import glob
import json
import os
import shutil
import statistics
import subprocess
import sys
import tempfile

ROOT = os.path.dirname(os.path.abspath(__file__))
LAYERS, M = 24, 8                       # bench.py's layer blobs and fold period
STEP_KERNELS = ('step_kernel', 'quad_kernel', 'pack_kernel', 'pack_v_kernel', 'pack_f_kernel', 'read_kernel')
SHADER_SETS = {
    'issue': ['SQ_WAVES', 'SQ_INSTS_VALU', 'SQ_INSTS_SALU', 'SQ_INSTS_LDS', 'SQ_INSTS_VMEM_RD', 'SQ_INSTS_VMEM_WR',
              'SQ_INSTS_SMEM', 'SQ_INSTS_MFMA'],
    'time': ['SQ_WAVE_CYCLES', 'SQ_BUSY_CYCLES', 'SQ_WAIT_ANY', 'SQ_WAIT_INST_ANY', 'SQ_ACTIVE_INST_VALU',
             'SQ_ACTIVE_INST_SCA', 'SQ_ACTIVE_INST_LDS', 'SQ_LDS_BANK_CONFLICT', 'GRBM_GUI_ACTIVE'],
    # the vector memory path of a compute unit: texture addresser busy (average over the units), L1 stalled on its
    # outstanding misses, L1 -> L2 read requests, addresser stalled by the L1
    'vmem': ['TA_BUSY_avr', 'TCP_PENDING_STALL_CYCLES_sum', 'TCP_TCC_READ_REQ_sum', 'TCP_TOTAL_CACHE_ACCESSES_sum',
             'TA_ADDR_STALLED_BY_TC_CYCLES_sum', 'GRBM_GUI_ACTIVE'],
    # instruction fetch: requests of the wavefronts, and the instruction caches' (one per two compute units) side
    'ifetch': ['SQ_IFETCH', 'SQC_ICACHE_REQ', 'SQC_ICACHE_HITS', 'SQC_ICACHE_MISSES', 'SQC_ICACHE_BUSY_CYCLES',
               'SQ_BUSY_CYCLES', 'GRBM_GUI_ACTIVE'],
}


def rocprof(args, bench_args, workdir, timeout=240):
    """One rocprofv3 run of bench.py; returns (command as text, directory with the csv output)."""
    out = tempfile.mkdtemp(prefix='prof_', dir=workdir)
    cmd = ['rocprofv3', *args, '--output-format', 'csv', '-d', out, '-o', 'p', '--',
           'python3', os.path.join(ROOT, 'bench.py'), *bench_args]
    env = dict(os.environ, TMPDIR='/tmp')
    r = subprocess.run(cmd, cwd='/tmp', env=env, capture_output=True, text=True, timeout=timeout)
    if r.returncode:
        sys.exit(f'{" ".join(cmd)}\nexit {r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-2000:]}')
    shown = ['rocprofv3', *args, '--output-format', 'csv', '-d', '<dir>', '-o', 'p', '--', 'python3', 'bench.py', *bench_args]
    return ' '.join(shown), out


def read_csv(d, suffix):
    rows = []
    for f in glob.glob(os.path.join(d, '**', '*' + suffix), recursive=True):
        rows += list(csv.DictReader(open(f)))
    return rows


def kind_of(i):
    return 'fold' if (i // LAYERS) % M == M - 1 else 'plain'


def counters(d, pick):
    """{(counter, kind): average per dispatch} over the dispatches whose kernel name `pick` accepts, in dispatch
    order; kind = fold / plain by the step of the period a dispatch belongs to ('all' for a calibration run)."""
    rows = [r for r in read_csv(d, 'counter_collection.csv') if pick(r['Kernel_Name'])]
    ids = sorted({int(r['Dispatch_Id']) for r in rows})
    pos = {x: i for i, x in enumerate(ids)}
    acc = collections.defaultdict(lambda: [0.0, 0])
    name = rows[0]['Kernel_Name'] if rows else ''
    for r in rows:
        for k in (kind_of(pos[int(r['Dispatch_Id'])]), 'all'):
            a = acc[(r['Counter_Name'], k)]
            a[0] += float(r['Counter_Value'])
            a[1] += 1
    return {k: v[0] / v[1] for k, v in acc.items()}, len(ids), name


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--workload', default='gdn-int8-g128')
    ap.add_argument('--out', default=os.path.join(ROOT, 'profiles'))
    ap.add_argument('--sets', default='trace,hbm,shader')
    ap.add_argument('--trace-steps', default='', metavar='K,W',
                    help="steps and warm-up of the trace pass instead of bench.py's own (e.g. 16,16)")
    ap.add_argument('--bench-args', default='', help='extra bench.py arguments, given as --bench-args=--mixed-fill')
    a = ap.parse_args()
    sets = a.sets.split(',')
    os.makedirs(a.out, exist_ok=True)
    work = tempfile.mkdtemp(prefix='profile_step_', dir='/tmp')
    targs = ['--workload', a.workload, '--no-cpu-baseline', *a.bench_args.split()]     # the trace: bench.py's own K, W
    bargs = [*targs, '--steps', str(2 * M), '--warmup', str(2 * M)]                   # counters: two fold periods
    if a.trace_steps:
        k, w = a.trace_steps.split(',')
        targs = [*targs, '--steps', k, '--warmup', w]
    names = STEP_KERNELS[:2]
    if '--op' in a.bench_args:                               # the prefill-side kernels instead
        names = ('read_kernel',) if 'read' in a.bench_args else STEP_KERNELS[2:5]
    is_step = lambda n: any(s in n for s in names)         # noqa: E731
    lines = [f'rocprofv3 profile of the decode-step kernel, bench.py workload {a.workload}'
             + (f' ({a.bench_args})' if a.bench_args else ''),
             f'made by: python profile_step.py --workload {a.workload} --sets {a.sets}'
             + (f' --trace-steps {a.trace_steps}' if a.trace_steps else '')
             + (f' --bench-args={a.bench_args}' if a.bench_args else ''),
             'every pass below is a run of its own, from /tmp with TMPDIR=/tmp; <dir> is a scratch directory', '']
    kernel = ''

    if 'trace' in sets:
        cmd, d = rocprof(['--kernel-trace', '--stats'], targs, work, timeout=600)
        rows = [r for r in read_csv(d, 'kernel_trace.csv') if is_step(r['Kernel_Name'])]
        rows.sort(key=lambda r: int(r['Start_Timestamp']))
        dur = [(int(r['End_Timestamp']) - int(r['Start_Timestamp'])) / 1e3 for r in rows]
        kernel = rows[0]['Kernel_Name']
        by = collections.defaultdict(list)
        for i, x in enumerate(dur):
            by[(i // LAYERS) % M].append(x)
        lines += ['== kernel trace ==', cmd, '', f'kernel: {kernel}',
                  f'dispatches {len(dur)}: average {statistics.mean(dur):.2f} us, median {statistics.median(dur):.2f} us',
                  f"registers as rocprofv3 prints them: VGPR_Count {rows[0].get('VGPR_Count')} "
                  f"(allocated unified registers / 2), Accum_VGPR_Count {rows[0].get('Accum_VGPR_Count')}, "
                  f"SGPR_Count {rows[0].get('SGPR_Count')}, LDS_Block_Size {rows[0].get('LDS_Block_Size')}, "
                  f"Scratch_Size {rows[0].get('Scratch_Size')}",
                  'duration by step of the fold period (the last one folds), us:']
        for k in sorted(by):
            lines.append(f'  step {k}: mean {statistics.mean(by[k]):7.2f}  min {min(by[k]):7.2f}  max {max(by[k]):7.2f}'
                         f'  n {len(by[k])}')
        stats = read_csv(d, 'kernel_stats.csv')
        lines += ['', 'rocprofv3 --stats, every kernel of the run (name, calls, total ns, average ns, %):']
        for r in stats[:6]:
            lines.append(f"  {r['Name'][:100]}  {r['Calls']}  {r['TotalDurationNs']}  {float(r['AverageNs']):.0f}  "
                         f"{float(r['Percentage']):.1f}")
        lines.append('')
        shutil.rmtree(d, ignore_errors=True)

    if 'hbm' in sets:
        lines.append('== HBM traffic ==')
        factor, per = {}, {}
        for c, known in (('FETCH_SIZE', 'bytes_read'), ('WRITE_SIZE', 'bytes_written')):
            cmd_c, d = rocprof(['--pmc', c], ['--calibrate-copy'], work)
            cal, ncal, kcal = counters(d, lambda n: 'copy' in n.lower())
            shutil.rmtree(d, ignore_errors=True)
            kib = cal[(c, 'all')]
            factor[c] = (1 << 30) / 1024 / kib                      # the copy moves 1 GiB each way per dispatch
            cmd_w, d = rocprof(['--pmc', c], bargs, work)
            val, n, kernel = counters(d, is_step)
            shutil.rmtree(d, ignore_errors=True)
            per[c] = {k: val[(c, k)] * 1024 * factor[c] for k in ('plain', 'fold', 'all')}
            lines += [cmd_c, f'  {kcal[:60]}: {ncal} copies of 1 GiB, {c} {kib:.1f} KiB per dispatch -> factor {factor[c]:.3f}',
                      cmd_w, f'  {n} dispatches; {c} KiB per dispatch: plain steps {val[(c, "plain")]:.1f}, fold steps '
                             f'{val[(c, "fold")]:.1f}']
        avg = {c: (per[c]['plain'] * (M - 1) + per[c]['fold']) / M for c in per}
        traffic = avg['FETCH_SIZE'] + avg['WRITE_SIZE']
        lines += ['scaled to bytes per launch:',
                  f"  plain step  read {per['FETCH_SIZE']['plain']:,.0f}  written {per['WRITE_SIZE']['plain']:,.0f}",
                  f"  fold step   read {per['FETCH_SIZE']['fold']:,.0f}  written {per['WRITE_SIZE']['fold']:,.0f}",
                  f'  average over a fold period of {M} steps: {traffic:,.0f} bytes per launch', '']
        path = os.path.join(a.out, 'hbm_traffic.json')
        kept = path if os.path.exists(path) else os.path.join(ROOT, 'profiles', 'hbm_traffic.json')
        table = json.load(open(kept)) if os.path.exists(kept) else {}          # other workloads' rows stay
        table[a.workload + (' ' + a.bench_args if a.bench_args else '')] = {
            'traffic': round(traffic), 'read_plain': round(per['FETCH_SIZE']['plain']),
            'read_fold': round(per['FETCH_SIZE']['fold']), 'written_plain': round(per['WRITE_SIZE']['plain']),
            'written_fold': round(per['WRITE_SIZE']['fold']), 'factor_fetch': round(factor['FETCH_SIZE'], 3),
            'factor_write': round(factor['WRITE_SIZE'], 3), 'kernel': kernel,
            'source': f'python profile_step.py --workload {a.workload} --sets hbm'}
        with open(path, 'w') as f:
            json.dump(table, f, indent=1, sort_keys=True)
            f.write('\n')

    if 'shader' in sets:
        lines.append('== shader counters, average per dispatch ==')
        for name, cs in SHADER_SETS.items():
            cmd, d = rocprof(['--pmc', *cs], bargs, work)
            val, n, kernel = counters(d, is_step)
            shutil.rmtree(d, ignore_errors=True)
            lines += [cmd, f'  {"counter":28s} {"plain step":>16s} {"fold step":>16s}']
            for c in cs:
                if (c, 'plain') in val:
                    lines.append(f'  {c:28s} {val[(c, "plain")]:16.1f} {val[(c, "fold")]:16.1f}')
            lines.append('')

    lines.insert(3, f'kernel: {kernel}')
    tag = a.workload + ('_' + a.bench_args.replace('--', '').replace(' ', '_') if a.bench_args else '')
    path = os.path.join(a.out, f'{tag}_step_kernel.txt')
    with open(path, 'w') as f:
        f.write('\n'.join(lines) + '\n')
    shutil.rmtree(work, ignore_errors=True)
    print(f'wrote {path}')


if __name__ == '__main__':
    main()
