"""Benchmark of the packed-state decode step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload gdn-int8-g128 | gdn-int8-g32 | gdn-int4-g64 | ...]

Headline workload (default): Gated DeltaNet decode at the Qwen3.5-4B shape -- 32 value / 16 key heads, d_k = d_v = 128,
256 slots, int8 state with one fp16 scale per (head, value row), int8 decode buffer of m = 8 tokens, bf16 q / k / v,
g and beta given -- on 24 independent layer blobs stepped back to back (3.6 GB of state, so no layer's state survives
in the 256 MiB Infinity Cache until its next step).  A "step" is one decode token through all 24 layers = 24 launches
of the fused step kernel through the C ABI (``SlotLayout.step`` -> ``sq_gdn_step``).  All slots start from a zero
state and advance in lockstep, so one step in m folds and re-quantizes every state tile (the reference's benchmark does
the same: benchmarks/decode_state.py:41-66 there times graphs of m steps = one fold).

Timing: whole fold periods only.  K and W are rounded up to multiples of m (``config.steps_requested`` keeps K;
``steps`` is what was timed), so every timed window holds exactly steps / m folds whatever K is.  The steps are
replayed from a HIP graph of m steps (m x 24 kernel nodes) unless ``--no-graph``.  Warm-up: one eager period, the
capture, and then at least MIN_WARM_PERIODS untimed replays of the graph whatever W says (``warmup`` in the line is
what was run: the first replay of a graph uploads it, and the clocks need a few milliseconds of load to settle), then
the timed periods between ``torch.cuda.synchronize()`` calls on the wall clock (``ms_per_step``, ``value``).  Every
timed period also has its own pair of HIP events on the launch stream: ``per_period_us`` lists them (microseconds per
launch), ``period_us`` holds their min / median / mean (the reference's benchmark reports the minimum over repeats of
the same graph, benchmarks/decode_state.py:41-66 there), and ``roofline`` is priced on their mean.

Prints ONE JSON line.  ``value`` = microseconds per layer per decode step (lower is better).  ``roofline`` prices the
step kernel against HBM: achieved = algorithmic state bytes per launch / average launch duration, where the
algorithmic bytes are (codes + scales) x (1 + 1/m) per slot (read every step, rewritten once per m steps) x slots.
``roofline.total`` prices the same duration against every byte the step has to move (state, live buffer slots,
appends, counters, inputs, output).  ``roofline.traffic`` is the HBM traffic per launch that profile_step.py measured
with rocprofv3 counters (read from profiles/hbm_traffic.json: a separate run, not this one; null if none).
``cpu_baseline`` times the CPU oracle (a torch restatement of the reference's own CPU path) on this box's host cores
on a bounded sample of the same workload, and ``cpu_baseline_c1`` the same oracle on the reference's own CPU-runnable
configuration (4 sequences, 4 / 2 heads, d 64, int8 group 64, bf16 buffer, m 8, 64 steps); reported baselines, not
targets.

Secondary figures: ``--workload`` (the other formats and families; ``gga4-pw8`` is the mixed-width GGA / STEP slot,
which re-fits every head at every token), ``--slots N`` (other batch sizes), ``--op write |
read`` (the prefill-side kernels), ``--mixed-fill`` (sequences of unequal lengths: every step folds 1/m of the slots),
``--fold-order`` (the step calls' optional dispatch order, for that case; the default run reports both as
``out_of_step``) and ``--calibrate-copy`` (the known-size copy that the HBM counters are scaled by).
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MIN_WARM_PERIODS = 8           # untimed graph replays before the clock starts (about 50 ms at the headline)
MAX_LISTED_PERIODS = 128       # per_period_us lists at most this many (the statistics use all)

WORKLOADS = {
    # name: (family, bits, group, hv, hk, dk, dv, slots, layers); group < 0: value-axis groups of -group rows;
    # bits 16: the unquantized bf16 state (the reference's control)
    'gdn-int8-g128': ('gdn', 8, 128, 32, 16, 128, 128, 256, 24),
    'gdn-int8-g32': ('gdn', 8, 32, 32, 16, 128, 128, 256, 24),
    'gdn-int4-g64': ('gdn', 4, 64, 32, 16, 128, 128, 256, 24),
    'gdn-int4-g32': ('gdn', 4, 32, 32, 16, 128, 128, 256, 24),
    'gdn-int4v-g32': ('gdn', 4, -32, 32, 16, 128, 128, 256, 24),
    'gdn-int8v-g32': ('gdn', 8, -32, 32, 16, 128, 128, 256, 24),
    'gdn-bf16': ('gdn', 16, 128, 32, 16, 128, 128, 256, 24),
    'gdn-olmo-int4-g64': ('gdn', 4, 64, 30, 30, 96, 192, 256, 24),        # OLMo-Hybrid-7B's layer: 30 heads, 96 x 192
    'mamba2-int8-g128': ('mamba2', 8, 128, 128, 8, 128, 64, 128, 24),
    'kda-int4-g32': ('kda', 4, 32, 32, 32, 128, 128, 256, 24),
    # Nemotron-3-Nano's layer (96 heads x head_dim 80 x d_state 128, 8 groups) and a d_state-256 layer (Falcon-H1 style)
    'mamba2-nano-int8-g128': ('mamba2', 8, 128, 96, 8, 128, 80, 128, 24),
    'mamba2-n256-int8-g128': ('mamba2', 8, 128, 128, 8, 256, 64, 64, 24),
    # the mixed-width GGA / STEP slot: bits = the plan's mean width, group = the FP8 window length
    'gga4-pw8': ('gga', 4, 8, 32, 16, 128, 128, 256, 24),
}


def workload_format(bits, group):
    """The oracle's / Quantizer's format triple of a workload, 'bf16' for the unquantized state."""
    return 'bf16' if bits == 16 else (bits, 'v' if group < 0 else 'k', abs(group))


def describe_state(bits, group):
    if bits == 16:
        return 'bf16, unquantized'
    return f'int{bits} {"value" if group < 0 else "key"}-axis group {abs(group)}, fp16 scales'


def measured_traffic(workload):
    """HBM bytes per launch (read + written, averaged over a fold period) that profile_step.py measured for the
    workload with rocprofv3 FETCH_SIZE / WRITE_SIZE, from the table it keeps; None if it holds no such row."""
    path = os.path.join(ROOT, 'profiles', 'hbm_traffic.json')
    if not os.path.exists(path):
        return None
    row = json.load(open(path)).get(workload)
    return row['traffic'] if row else None


def stored_bytes_per_slot(bits, group, hv, dk, dv):
    codes = hv * dv * dk * bits // 8
    if bits == 16:
        return codes
    scales = hv * (dv // -group) * dk * 2 if group < 0 else hv * dv * (-(-dk // group)) * 2
    return codes + scales


def state_bytes_per_slot(bits, group, hv, dk, dv, m):
    return stored_bytes_per_slot(bits, group, hv, dk, dv) * (1 + 1 / m)


def total_bytes_per_slot(fam, bits, group, hv, hk, dk, dv, m, in_bytes=2, out_bytes=2, be=1):
    """Every byte one decode step of one slot has to move, averaged over a fold period: the state as above; the live
    part of the decode buffer ((m - 1) / 2 slots on average: values, keys, their scales, cumulative decays); the
    append of one slot; counters and running decay read and written; the token's inputs and its output.  KDA keeps
    the decays per key channel (fp32 [m, d_k] per head), which is why its total is far above its state bytes."""
    live = (m - 1) / 2
    gdim = dk if fam == 'kda' else 1                          # decay entries per (head, slot)
    per_slot = hv * dv * be + hk * dk * be + (hv + hk) * 2 + hv * gdim * 4      # one buffer slot: u, k, scales, G
    counters = 2 * (hv * gdim * 4 + hv * 4)                                     # GCUR, NPTR: read + write
    if fam == 'gdn':
        inputs = 2 * hk * dk * in_bytes + hv * dv * in_bytes + 2 * hv * 4
    elif fam == 'kda':
        inputs = 2 * hv * dk * in_bytes + hv * dk * 4 + hv * dv * in_bytes + hv * 4
    else:
        inputs = 2 * hk * dk * in_bytes + hv * dv * in_bytes + hv * 4 + 3 * hv * 4 / 128
    return (state_bytes_per_slot(bits, group, hv, dk, dv, m) + live * per_slot + per_slot + counters + inputs
            + hv * dv * out_bytes)


def build(workload, m, device):
    import statequant_amd as sq
    from statequant_amd.kernels import KDASlotLayout, Mamba2SlotLayout, SlotLayout
    fam, bits, group, hv, hk, dk, dv, slots, layers = WORKLOADS[workload]
    fmt = workload_format(bits, group)
    fmt = fmt if fmt == 'bf16' else sq.Quantizer(*fmt)
    if fam == 'gdn':
        lay = SlotLayout(fmt, hv, hk, dk, dv, m=m, buffer_bits=8)
    elif fam == 'kda':
        lay = KDASlotLayout(fmt, hv, dk, dv, m=m, buffer_bits=8)
    else:
        lay = Mamba2SlotLayout(fmt, hv, hk, dk, dv, m=m, buffer_bits=8)
    blobs = [lay.alloc(slots + 1, device) for _ in range(layers)]            # slot 0 is the engine's null slot
    views = [lay.views(b) for b in blobs]
    gen = torch.Generator(device='cpu').manual_seed(0)
    idx = (torch.randperm(slots, generator=gen) + 1).to(torch.int32).to(device)
    return fam, lay, views, idx


def make_inputs(fam, lay, slots, layers, m, device, seed=1):
    """Synthetic inputs of one fold period: a distinct set per (step in period, layer), in the configs' distributions."""
    gen = torch.Generator(device=device).manual_seed(seed)
    r = lambda *s: torch.randn(*s, device=device, generator=gen)          # noqa: E731
    hv, hk, dk, dv = lay.HV, lay.HK, lay.DK, lay.DV
    out = []
    for _ in range(m * layers):
        if fam == 'gdn':
            out.append(dict(q=r(slots, hk, dk).bfloat16(), k=r(slots, hk, dk).bfloat16(), v=r(slots, hv, dv).bfloat16(),
                            g=-torch.nn.functional.softplus(r(slots, hv)), beta=torch.sigmoid(r(slots, hv))))
        elif fam == 'kda':
            out.append(dict(q=r(slots, hv, dk).bfloat16(), k=r(slots, hv, dk).bfloat16(), v=r(slots, hv, dv).bfloat16(),
                            g=-torch.nn.functional.softplus(r(slots, hv, dk)), beta=torch.sigmoid(r(slots, hv))))
        else:
            out.append(dict(x=r(slots, hv, dv).bfloat16(), dt=r(slots, hv) * 0.5 - 2, B=r(slots, hk, dk).bfloat16(),
                            C=r(slots, hk, dk).bfloat16()))
    extra = {}
    if fam == 'mamba2':
        extra = dict(A=-torch.exp(torch.rand(hv, device=device, generator=gen) * 2), D=r(hv), dt_bias=r(hv) * 0.1)
    return out, extra


def launch(fam, lay, views, idx, inp, extra, out, order=None):
    if fam == 'gdn':
        lay.step(views, idx, inp['q'], inp['k'], inp['v'], out, lay.DK ** -0.5, g=inp['g'], beta=inp['beta'],
                 order=order)
    elif fam == 'kda':
        lay.step(views, idx, inp['q'], inp['k'], inp['v'], inp['g'], inp['beta'], out, order=order)
    else:
        lay.step(views, idx, inp['x'], inp['dt'], inp['B'], inp['C'], out, extra['A'], extra['D'], extra['dt_bias'],
                 order=order)


def timed_periods(stream, run_period, warm_periods, periods):
    """`warm_periods` untimed calls of `run_period()`, then `periods` timed ones on `stream`: the wall clock around
    all of them between device synchronisations, and one HIP event between every two periods.  Returns (wall seconds,
    [milliseconds of each period])."""
    for _ in range(warm_periods):
        run_period()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(periods + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev[0].record(stream)
    for i in range(periods):
        run_period()
        ev[i + 1].record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, [ev[i].elapsed_time(ev[i + 1]) for i in range(periods)]


def out_of_step_figures(fam, lay, views, idx, inputs, extra, out, m, layers, slots, stream, dev, periods=16):
    """Secondary figures of the default run: the same launches with the fill levels dealt at random over the batch
    rows (--mixed-fill), in batch order and in the order of `fold_order` (its launch included); us per launch."""
    gen = torch.Generator().manual_seed(2)
    fill = (torch.arange(slots, dtype=torch.int32) % m)[torch.randperm(slots, generator=gen)].to(dev)[:, None]
    order = torch.zeros(slots, dtype=torch.int32, device=dev)
    res = {}
    with torch.cuda.stream(stream):
        for name, ordered in (('batch_order_us', False), ('fold_order_us', True)):
            stream.synchronize()
            for V in views:
                V['NPTR'][idx.long()] = fill.expand(slots, V['NPTR'].shape[1])

            def period():
                for s in range(m):
                    if ordered:
                        lay.fold_order(views[0], idx, out=order)
                    for L in range(layers):
                        launch(fam, lay, views[L], idx, inputs[s * layers + L], extra, out, order if ordered else None)

            period()
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                period()
            _, per_ms = timed_periods(stream, graph.replay, 4, periods)
            res[name] = round(sum(per_ms) * 1e3 / (periods * m * layers), 3)
    res['what'] = ('sequences out of step: 1/m of the slots fold on every step, fill levels dealt at random over the '
                   'rows (--mixed-fill); fold_order_us: dispatched in the order of sq_fold_order, one list per decode '
                   'step, its launch inside the timed region (--fold-order)')
    return res


def period_stats(per_ms, launches_per_period):
    """Per-launch microseconds of every timed period and their min / median / mean."""
    us = sorted(x * 1e3 / launches_per_period for x in per_ms)
    n = len(us)
    med = us[n // 2] if n % 2 else 0.5 * (us[n // 2 - 1] + us[n // 2])
    listed = [round(x * 1e3 / launches_per_period, 3) for x in per_ms[:MAX_LISTED_PERIODS]]
    return listed, {'min': round(us[0], 3), 'median': round(med, 3), 'mean': round(sum(us) / n, 3), 'periods': n}


def cpu_baseline(workload, m, budget_s=20.0):
    """The CPU oracle on a bounded sample of the workload: one layer, all slots, one fold period (m steps incl. the
    fold), repeated while the budget lasts.  Returns the JSON object."""
    from oracle import states as ST
    fam, bits, group, hv, hk, dk, dv, slots, layers = WORKLOADS[workload]
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    gen = torch.Generator().manual_seed(0)
    r = lambda *s: torch.randn(*s, generator=gen)          # noqa: E731
    S0 = r(slots * hv, dv, dk) * 0.1
    fmt = workload_format(bits, group)
    if fam == 'gdn':
        st = ST.GDNOracle(S0, fmt, m=m, hv=hv, hk=hk, buffer_bits=8)
    elif fam == 'kda':
        st = ST.KDAOracle(S0, fmt, m=m, hv=hv, buffer_bits=8)
    else:
        st = ST.Mamba2Oracle(S0, fmt, m=m, hv=hv, hk=hk, buffer_bits=8)
        A, D, dtb = -torch.exp(torch.rand(hv, generator=gen) * 2), r(hv), r(hv) * 0.1
    steps, t_total = 0, 0.0
    while t_total < budget_s and steps < 4 * m:
        for _ in range(m):
            if fam == 'gdn':
                args = (r(slots * hk, dk).bfloat16(), r(slots * hk, dk).bfloat16(), r(slots * hv, dv).bfloat16(),
                        -torch.nn.functional.softplus(r(slots * hv)), torch.sigmoid(r(slots * hv)), dk ** -0.5)
            elif fam == 'kda':
                args = (r(slots * hv, dk).bfloat16(), r(slots * hv, dk).bfloat16(), r(slots * hv, dv).bfloat16(),
                        -torch.nn.functional.softplus(r(slots * hv, dk)), torch.sigmoid(r(slots * hv)))
            else:
                args = (r(slots, hv, dv).bfloat16(), r(slots, hv) * 0.5 - 2, r(slots, hk, dk).bfloat16(),
                        r(slots, hk, dk).bfloat16(), A, D, dtb, True, None)
            t0 = time.perf_counter()
            st.step(*args)
            t_total += time.perf_counter() - t0
            steps += 1
    return {'value': round(t_total / steps * 1e6, 1), 'unit': 'us per layer-step', 'cores': cores, 'kind': 'port',
            'sample': f'{workload}: 1 layer x {slots} slots, {steps} steps ({steps // m} fold periods of m={m}), '
                      f'torch CPU oracle, {cores} threads'}


def cpu_baseline_c1():
    """The CPU oracle on the reference's own CPU-runnable configuration, whole: 4 sequences, 4 value / 2 key heads,
    d_k = d_v = 64, int8 state in groups of 64, bf16 decode buffer of m = 8, 64 steps from a zero state, seed 0."""
    from oracle import states as ST
    B, hv, hk, d, m, steps = 4, 4, 2, 64, 8, 64
    torch.set_num_threads(1)
    gen = torch.Generator().manual_seed(0)
    r = lambda *s: torch.randn(*s, generator=gen)          # noqa: E731
    st = ST.GDNOracle(torch.zeros(B * hv, d, d), (8, 'k', 64), m=m, hv=hv, hk=hk, buffer_bits=16)
    t_total = 0.0
    for _ in range(steps):
        args = (r(B * hk, d).bfloat16(), r(B * hk, d).bfloat16(), r(B * hv, d).bfloat16(),
                -torch.nn.functional.softplus(r(B * hv)), torch.sigmoid(r(B * hv)), d ** -0.5)
        t0 = time.perf_counter()
        st.step(*args)
        t_total += time.perf_counter() - t0
    torch.set_num_threads(os.cpu_count() or 1)
    return {'value': round(t_total / steps * 1e6, 1), 'unit': 'us per layer-step', 'cores': 1, 'kind': 'port',
            'sample': f'reference CPU case: {B} sequences x {hv}/{hk} heads x {d} x {d}, int8 g64, bf16 buffer, m={m}, '
                      f'{steps} steps from zero, torch CPU oracle, 1 thread'}


def gga_plan(hv, dk, layers, seed=0):
    """A synthetic plan at a mean of 4 bits with one fp16 pivot per layer (charged 8 bits, as the method's allocator
    does): 12 x 2, 11 x 4, 6 x 6, 2 x 8 bits and the pivot over the 32 heads, shuffled per layer."""
    from statequant_amd.kernels.gga import GGAPlan
    gen = torch.Generator().manual_seed(seed)
    base = [2] * 12 + [4] * 11 + [6] * 6 + [8] * 2 + [16]
    base = (base * (-(-hv // len(base))))[:hv]
    return GGAPlan({L: (torch.tensor(base)[torch.randperm(hv, generator=gen)], torch.rand(hv, dk, generator=gen) + 0.5)
                    for L in range(layers)})


def gga_bytes_per_slot_step(pk, layer):
    """Algorithmic bytes of one token on one slot of one layer: every head read and re-written at its width; per
    non-pivot head the full window read, its left factors re-written, one new pair written."""
    from statequant_amd.kernels.gga import head_bytes
    widths = pk.tables[layer][1]
    st = 2 * sum(head_bytes(b, pk.DK, pk.DV) for b in widths)
    nonp = sum(b != 16 for b in widths)
    win = nonp * (pk.m * (pk.DK + pk.DV + 8) + pk.m * (pk.DK + 4) + pk.DK + pk.DV + 8) if pk.pw else 0
    return st + win


def bench_gga(a, dev):
    """The GGA / STEP slot step (GGAPacked.step -> sq_gga_step) at the Qwen3.5-4B GDN shape: every token re-fits and
    re-packs every head, so the state is read and written on every step."""
    from statequant_amd.kernels.gga import GGAPacked
    fam, bits, m, hv, hk, dk, dv, slots, layers = WORKLOADS[a.workload]
    pk = GGAPacked(gga_plan(hv, dk, layers), hv, hk, dk, dv, pw=True, m=m).prepare(dev)
    views = [pk.views(pk.alloc(slots + 1, dev)) for _ in range(layers)]
    gen = torch.Generator(device=dev).manual_seed(1)
    r = lambda *s: torch.randn(*s, device=dev, generator=gen)          # noqa: E731
    idx = (torch.randperm(slots, generator=torch.Generator().manual_seed(0)) + 1).to(torch.int32).to(dev)
    for L in range(layers):
        pk.write(views[L], idx, r(slots, hv, dv, dk) * 0.3, layer=L)
    A_log, dtb = r(hv) * 0.3, r(hv) * 0.3
    period_len = 8
    inputs = [dict(q=r(slots, hk, dk).bfloat16(), k=r(slots, hk, dk).bfloat16(), v=r(slots, hv, dv).bfloat16(),
                   a=r(slots, hv) * 0.5 - 2, b=r(slots, hv)) for _ in range(period_len * layers)]
    out = torch.zeros(slots, hv, dv, device=dev, dtype=torch.bfloat16)

    def period():
        for s in range(period_len):
            for L in range(layers):
                i = inputs[s * layers + L]
                pk.step(views[L], idx, i['q'], i['k'], i['v'], out, dk ** -0.5, gate=(i['a'], i['b'], A_log, dtb), layer=L)

    requested = (a.steps, a.warmup)
    a.steps = max(-(-a.steps // period_len), 1) * period_len          # whole graphs of period_len steps
    use_graph = not a.no_graph
    torch.cuda.synchronize()                                # states and inputs were made on the default stream
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        period()
        stream.synchronize()
        if use_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                period()
            run_period = graph.replay
        else:
            run_period = period
        warm = max(-(-a.warmup // period_len) - 1, 2)
        wall, per_ms = timed_periods(stream, run_period, warm, a.steps // period_len)
    a.warmup = (warm + 1) * period_len
    per_period_us, pstats = period_stats(per_ms, period_len * layers)
    steps = a.steps
    assert torch.isfinite(out.float()).all(), 'non-finite output'
    n_launch = steps * layers
    us_wall, us_kernel = wall * 1e6 / n_launch, sum(per_ms) * 1e3 / n_launch
    alg = sum(gga_bytes_per_slot_step(pk, L) for L in range(layers)) / layers * slots
    achieved = alg / (us_kernel * 1e-6) / 1e9
    res = {
        'metric': 'us_per_layer_decode_step', 'value': round(us_wall, 3), 'unit': 'us',
        'n_gpus': 1, 'steps': steps, 'warmup': a.warmup, 'ms_per_step': round(wall * 1e3 / steps, 5),
        'higher_is_better': False, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': a.workload, 'family': 'gdn (GGA / STEP slot)', 'slots': slots, 'layers': layers,
                   'value_heads': hv, 'key_heads': hk, 'd_k': dk, 'd_v': dv,
                   'state': f'per-head widths 2/4/6/8 bit + one fp16 pivot per layer, {pk.bits_per_value():.3f} bits '
                            f'per value with the window', 'window': f'FP8 pairs, m={m}', 'inputs': 'bf16',
                   'launch': 'hip-graph' if use_graph else 'eager', 'steps_requested': requested[0],
                   'warmup_requested': requested[1], 'steps_timed': steps, 'folds_timed': None,
                   'bytes_per_slot': pk.nbytes,
                   'algorithmic_bytes_per_slot_step': round(alg / slots)},
        'hbm_gbs': round(achieved, 1),
        'period_us': pstats, 'per_period_us': per_period_us,
        'roofline': {'bound': 'hbm', 'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                     'frac': round(achieved / HBM_PEAK_GBS, 4), 'traffic': measured_traffic(a.workload),
                     'traffic_source': 'profiles/hbm_traffic.json (rocprofv3 run of profile_step.py, not this run)',
                     'kernel_us': round(us_kernel, 3), 'algorithmic_bytes_per_launch': round(alg)},
    }
    if not a.no_cpu_baseline:
        res['cpu_baseline'] = cpu_baseline_gga(a.workload, a.cpu_budget)
    print(json.dumps(res))


def cpu_baseline_gga(workload, budget_s=20.0):
    """The CPU oracle of the GGA slot step on a bounded sample: one layer, 32 slots."""
    from oracle import gga as G
    fam, bits, m, hv, hk, dk, dv, slots, layers = WORKLOADS[workload]
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    n = min(slots, 32)
    plan = gga_plan(hv, dk, 1)
    b, w = plan.plan[0]
    gen = torch.Generator().manual_seed(0)
    r = lambda *s: torch.randn(*s, generator=gen)          # noqa: E731
    st = G.GGAState(b, w, n + 1, hv, hk, dk, dv, pw=True, m=m)
    idx = torch.arange(1, n + 1, dtype=torch.int32)
    st.write(idx, r(n, hv, dk, dv) * 0.3)
    steps, t_total = 0, 0.0
    while t_total < budget_s and steps < 16:
        args = (r(n, hk, dk).bfloat16(), r(n, hk, dk).bfloat16(), r(n, hv, dv).bfloat16(), dk ** -0.5,
                -torch.nn.functional.softplus(r(n, hv)), torch.sigmoid(r(n, hv)))
        t0 = time.perf_counter()
        st.step(idx, *args)
        t_total += time.perf_counter() - t0
        steps += 1
    return {'value': round(t_total / steps * 1e6 * slots / n, 1), 'unit': 'us per layer-step', 'cores': cores,
            'kind': 'port', 'sample': f'{workload}: 1 layer x {n} of {slots} slots (time scaled by {slots // n}), '
                                      f'{steps} steps, torch CPU oracle, {cores} threads'}


def calibrate_copy(dev, nbytes=1 << 30, reps=20):
    """`reps` plain copies of `nbytes` (reads nbytes, writes nbytes each): the reference point for the HBM counters."""
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    dst.copy_(src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / reps
    print(json.dumps({'calibrate_copy': True, 'bytes_read': nbytes, 'bytes_written': nbytes, 'copies': reps + 1,
                      'us_per_copy': round(us, 2), 'gbs_read_plus_write': round(2 * nbytes / us * 1e-3, 1)}))


def bench_convert(a, lay, views, idx, dev):
    """`SlotLayout.write` (fp32 state -> codes + scales, buffers emptied) or `.read` (stored state advanced across
    the pending buffer -> fp32) over all slots of every layer blob; one launch per layer.  Algorithmic bytes: the fp32
    state on one side (4 bytes per code) plus codes and scales on the other."""
    fam, bits, group, hv, hk, dk, dv, slots, layers = WORKLOADS[a.workload]
    S = torch.randn(slots, hv, dv, dk, device=dev) * 0.3
    idl = idx.long()
    for V in views:                                         # a defined state with a partly filled buffer
        lay.write(V, idl, S)
        V['NPTR'][idl] = 3
        V['GB'][idl] = -torch.rand_like(V['GB'][idl])
        V['GCUR'][idl] = -torch.rand_like(V['GCUR'][idl]) - 1.0
        V['KB'][idl] = torch.randint(-100, 100, V['KB'][idl].shape, device=dev).to(V['KB'].dtype)
        V['UB'][idl] = torch.randint(-100, 100, V['UB'][idl].shape, device=dev).to(V['UB'].dtype)
        V['KBS'][idl] = 0.01
        V['UBS'][idl] = 0.01
    run = (lambda V: lay.write(V, idl, S)) if a.op == 'write' else (lambda V: lay.read(V, idl))
    reps = max(a.steps // 64, 4)
    for V in views:
        run(V)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(reps):
        for V in views:
            run(V)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    n = reps * layers
    us = e0.elapsed_time(e1) * 1e3 / n
    alg = slots * (hv * dv * dk * 4 + stored_bytes_per_slot(bits, group, hv, dk, dv))
    print(json.dumps({
        'metric': f'us_per_layer_{a.op}', 'value': round(wall * 1e6 / n, 3), 'unit': 'us', 'n_gpus': 1, 'steps': reps,
        'warmup': 1, 'higher_is_better': False, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': a.workload, 'op': a.op, 'slots': slots, 'layers': layers,
                   'includes': 'host-side index conversion and output allocation of SlotLayout.' + a.op},
        'roofline': {'bound': 'hbm', 'achieved': round(alg / us * 1e-3, 1), 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                     'frac': round(alg / us * 1e-3 / HBM_PEAK_GBS, 4), 'traffic': None, 'kernel_us': round(us, 3),
                     'algorithmic_bytes_per_launch': alg}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=1024)
    ap.add_argument('--warmup', type=int, default=512)
    ap.add_argument('--workload', default='gdn-int8-g128', choices=list(WORKLOADS))
    ap.add_argument('--m', type=int, default=8)
    ap.add_argument('--slots', type=int, default=None,
                    help='number of sequences instead of the workload\'s own (the reference quotes batch 128 and 512)')
    ap.add_argument('--no-graph', action='store_true', help='launch eagerly instead of replaying a HIP graph')
    ap.add_argument('--mixed-fill', action='store_true',
                    help='start the slots with 0 .. m - 1 tokens in their buffers, 1/m of them each, dealt at random over '
                         'the batch rows, so that every step folds 1/m of the slots (sequences of unequal lengths, as '
                         'a serving engine has them) instead of all slots folding on the same step; a secondary '
                         'figure, the headline is the lockstep configuration')
    ap.add_argument('--fold-order', action='store_true',
                    help='dispatch every decode step in the order of `fold_order` (one small launch per step, inside '
                         'the timed region, whose list serves the 24 layer launches): the rows that fold on the step '
                         'spread evenly over the launch.  An addition to the reference\'s interface, for sequences '
                         'out of step (--mixed-fill)')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--instances', default='', metavar='LIST',
                    help='comma-separated exclusions handed to sq_debug_select, for same-machine comparisons of the '
                         'kernel instances that can serve the workload: no-specialised, no-group, '
                         'lds-pad=<bytes> (unused dynamic LDS per workgroup: fewer resident workgroups)')
    ap.add_argument('--cpu-budget', type=float, default=20.0)
    ap.add_argument('--op', default='step', choices=['step', 'write', 'read'],
                    help="step: the decode step (the headline); write / read: the prefill-side pack and read kernels "
                         "on the same slots (SlotLayout.write / .read)")
    ap.add_argument('--calibrate-copy', action='store_true',
                    help='instead of the workload, run plain device copies of 1 GiB (the known-size kernel that '
                         'rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by) and print their rate')
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit('bench.py: this build measures one GPU; the decode step has no cross-GPU exchange (slots shard '
                 'freely), so a multi-GPU figure would be N independent copies of this run. Use --gpus 1.')
    if not torch.cuda.is_available():
        sys.exit('bench.py: no GPU visible; the packed decode step only runs as HIP kernels')
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    if a.calibrate_copy:
        return calibrate_copy(dev)
    if a.instances:
        from statequant_amd.kernels import _hip
        off = {x.strip() for x in a.instances.split(',') if x.strip()}
        pad = sum(int(x.split('=')[1]) for x in off if x.startswith('lds-pad='))
        assert {x for x in off if not x.startswith('lds-pad=')} <= {'no-specialised', 'no-group'}, off
        _hip.select_instances(no_specialised='no-specialised' in off, no_group_kernel='no-group' in off, lds_pad_bytes=pad)
    m = a.m
    if a.slots:
        w = WORKLOADS[a.workload]
        WORKLOADS[a.workload] = w[:7] + (a.slots,) + w[8:]
    fam, bits, group, hv, hk, dk, dv, slots, layers = WORKLOADS[a.workload]
    if fam == 'gga':
        return bench_gga(a, dev)
    fam, lay, views, idx = build(a.workload, m, dev)
    if a.op != 'step':
        return bench_convert(a, lay, views, idx, dev)
    inputs, extra = make_inputs(fam, lay, slots, layers, m, dev)
    if a.mixed_fill:
        gen = torch.Generator().manual_seed(2)
        fill = (torch.arange(slots, dtype=torch.int32) % m)[torch.randperm(slots, generator=gen)].to(dev)[:, None]
        for V in views:
            V['NPTR'][idx.long()] = fill.expand(slots, V['NPTR'].shape[1])
    out = torch.zeros(slots, hv, dv, device=dev, dtype=torch.bfloat16)

    order = torch.zeros(slots, dtype=torch.int32, device=dev) if a.fold_order else None

    def period():                                           # m steps x layers launches
        for s in range(m):
            if order is not None:                           # one list per decode step, from the first layer's counters
                lay.fold_order(views[0], idx, out=order)
            for L in range(layers):
                launch(fam, lay, views[L], idx, inputs[s * layers + L], extra, out, order)

    requested = (a.steps, a.warmup)
    a.steps = max(-(-a.steps // m), 1) * m                  # whole fold periods, so that any K times steps / m folds
    use_graph = not a.no_graph
    torch.cuda.synchronize()                                # states and inputs were made on the default stream
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        period()                                            # one eager period first (module load etc.)
        stream.synchronize()
        if use_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                period()
            run_period = graph.replay
        else:
            run_period = period
        warm = max(-(-a.warmup // m) - 1, MIN_WARM_PERIODS)  # untimed periods on the timed path itself
        wall, per_ms = timed_periods(stream, run_period, warm, a.steps // m)
    a.warmup = (warm + 1) * m                               # steps run before the clock started
    ev_ms = sum(per_ms)
    per_period_us, pstats = period_stats(per_ms, m * layers)
    assert torch.isfinite(out.float()).all(), 'non-finite output'
    n_launch = a.steps * layers
    us_wall = wall * 1e6 / n_launch
    us_kernel = ev_ms * 1e3 / n_launch                      # average launch-to-launch duration on the stream
    alg_bytes = state_bytes_per_slot(bits, group, hv, dk, dv, m) * slots
    achieved = alg_bytes / (us_kernel * 1e-6) / 1e9
    tot_bytes = total_bytes_per_slot(fam, bits, group, hv, hk, dk, dv, m) * slots
    tot_gbs = tot_bytes / (us_kernel * 1e-6) / 1e9
    res = {
        'metric': 'us_per_layer_decode_step', 'value': round(us_wall, 3), 'unit': 'us',
        'n_gpus': 1, 'steps': a.steps, 'warmup': a.warmup, 'ms_per_step': round(wall * 1e3 / a.steps, 5),
        'higher_is_better': False, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': a.workload, 'family': fam, 'slots': slots, 'layers': layers, 'value_heads': hv,
                   'key_heads': hk, 'd_k': dk, 'd_v': dv, 'state': describe_state(bits, group),
                   'buffer': f'int8, m={m}', 'inputs': 'bf16', 'launch': 'hip-graph' if use_graph else 'eager',
                   'steps_requested': requested[0], 'warmup_requested': requested[1], 'steps_timed': a.steps,
                   'folds_timed': a.steps // m if not a.mixed_fill else None,
                   'fold_schedule': 'mixed (1/m of the slots per step)' if a.mixed_fill else 'lockstep',
                   'dispatch_order': 'fold_order' if a.fold_order else 'batch order',
                   'instances_excluded': a.instances or None,
                   'state_bytes_per_slot_step': round(state_bytes_per_slot(bits, group, hv, dk, dv, m))},
        'hbm_gbs': round(achieved, 1),
        'period_us': pstats, 'per_period_us': per_period_us,
        'roofline': {'bound': 'hbm', 'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                     'frac': round(achieved / HBM_PEAK_GBS, 4), 'traffic': measured_traffic(a.workload),
                     'traffic_source': 'profiles/hbm_traffic.json (rocprofv3 run of profile_step.py, not this run)',
                     'kernel_us': round(us_kernel, 3), 'algorithmic_bytes_per_launch': round(alg_bytes),
                     'total': {'bytes_per_launch': round(tot_bytes), 'achieved': round(tot_gbs, 1),
                               'frac': round(tot_gbs / HBM_PEAK_GBS, 4),
                               'counts': 'state + live buffer slots + append + counters + inputs + output'}},
    }
    if use_graph and not a.mixed_fill and not a.fold_order and hasattr(lay, 'fold_order'):
        res['out_of_step'] = out_of_step_figures(fam, lay, views, idx, inputs, extra, out, m, layers, slots, stream, dev)
    if not a.no_cpu_baseline:
        res['cpu_baseline'] = cpu_baseline(a.workload, m, a.cpu_budget)
        res['cpu_baseline_c1'] = cpu_baseline_c1()
    print(json.dumps(res))


if __name__ == '__main__':
    main()
