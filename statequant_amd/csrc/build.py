"""Build libsqhip.so (the C-ABI library of include/statequant_hip.h) for gfx950 with hipcc.

    python -m statequant_amd.csrc.build [-j N] [--force] [--timeline] [--resources [PATTERN]]

The step kernels are templates on (bits, d_k, d_v, group, int8-buffer, max m).  ``CASES`` below lists the instances
that are compiled; this script writes one small translation unit per chunk of instances plus the dispatch table into
``csrc/build/`` (not tracked), compiles them in parallel and links ``statequant_amd/libsqhip.so`` next to the Python
package, where the loader looks for it.  hipcc cross-compiles, so no GPU is needed to build.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import hashlib
import itertools
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
OUT = os.path.join(HERE, 'build')
LIB = os.path.join(PKG, 'libsqhip.so')
ARCH = 'gfx950'

# -ffp-contract=off: every fused multiply-add in the kernels is written explicitly, as in the reference's kernels.
# The packed-fp32 target feature is switched off on purpose (plain v_fma / v_mul only).
HIPCC_FLAGS = ['--offload-arch=' + ARCH, '-O3', '-std=c++17', '-fPIC', '-ffp-contract=off',
               '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops', '-Wno-unused-command-line-argument',
               # scalar kernel arguments ahead of a parameter struct arrive in registers (no load at wave start)
               '-mllvm', '-amdgpu-kernarg-preload-count=16']


def _cases():
    """family -> [(bits, dk, dv, group, qbuf, mmax, axv)].  Shapes: Qwen3.5 GDN 128x128, small test heads 64x64,
    OLMo-Hybrid 96x192, a 96x96 head, 128x256 (the power-of-two problem that 96x192 pads to); Mamba2 d_state 128 /
    head_dim 64 (Nemotron-H), 128 x 128, 64 x 64, d_state 256 / head_dim 64 (Falcon-H1; key-axis groups and bf16 only), d_state 128 / head_dim 80 (Nemotron-3-Nano) and 96 / 80 (the
    reference tests' odd head);
    KDA 128x128, 96x96, 64x64, 128x256 and 64x32 (the reference tests' wide and small heads).  Key-axis groups: every power of two from 32 up to the padded d_k."""
    shapes = {
        'gdn': [(128, 128), (64, 64), (96, 192), (96, 96), (128, 256)],
        'mamba2': [(128, 64), (128, 128), (64, 64), (128, 80), (96, 80), (256, 64)],
        'kda': [(128, 128), (96, 96), (64, 64), (128, 256), (64, 32)],
    }
    out = {}
    for fam, shp in shapes.items():
        rows = []
        for (dk, dv), bits, qbuf in itertools.product(shp, (8, 4), (1, 0)):
            dkp = 1 << (dk - 1).bit_length()
            for group in (32, 64, 128):
                if group > dkp:
                    continue
                rows.append((bits, dk, dv, group, qbuf, 8, 0))
                rows.append((bits, dk, dv, group, qbuf, 16, 0))      # a buffer of up to 16 tokens
            for mmax in (8, 16) if dk <= 128 else ():                # value-axis groups: d_k up to 128
                if dv % 32 == 0:
                    rows.append((bits, dk, dv, 32, qbuf, mmax, 1))   # value-axis groups of 32 rows
                if dv % 64 == 0:
                    rows.append((bits, dk, dv, 64, qbuf, mmax, 1))   # ... of 64 rows
                if fam != 'gdn' or (dk, dv) in ((128, 128), (64, 64)):
                    rows.append((bits, dk, dv, 16, qbuf, mmax, 1))   # ... and of 16 (the reference's KDA / Mamba2 tests)
        for (dk, dv), qbuf in itertools.product(shp, (1, 0)):        # the unquantized control: bf16 (GDN also fp32) state
            for mmax in (8, 16):
                rows.append((16, dk, dv, dk, qbuf, mmax, 0))
                if fam == 'gdn':
                    rows.append((32, dk, dv, dk, qbuf, mmax, 0))
        out[fam] = rows
    return out


CASES = _cases()
GGA_SHAPES = [(128, 128), (64, 64)]                  # (d_k, d_v) of the mixed-width GGA / STEP slot (sq_gga.cuh)
PARAMS = {'gdn': 'GdnParams', 'kda': 'KdaParams', 'mamba2': 'Mamba2Params'}
# families with a workgroup-per-key-head kernel (sq_<family>_quad.cuh) -> value heads per workgroup that are built
QUAD_FAMILIES = {'gdn': (2, 1), 'mamba2': (4, 2, 1)}
# compile-time specialisations of the step kernels (SPEC, sq_params.h), most specific first; 0: everything read from
# the arguments.  Built for the default buffer (int8, 8 tokens) only.
SPECS = {'gdn': (1, 2, 0), 'kda': (1, 0), 'mamba2': (1, 0)}


def specs_of(fam, c, quad):
    """SPEC values an instance is built for: the workgroup-per-key-head kernels for every case they serve, the
    one-wavefront kernels for the cases that have no such kernel."""
    bits, dk, dv, group, qbuf, mmax, axv = c
    if not (qbuf and mmax == 8) or (not quad and quad_variants(fam, c)):
        return (0,)
    if not quad and fam != 'kda':
        # measured on the one-wavefront kernels: KDA int4 g32 40.0 -> 38.9 us, GDN value-axis int4 36.3 -> 35.1, but
        # value-axis int8 45.2 -> 48.4 and Mamba2 d_state 256 41.9 -> 48.1 (their register allocation tips over)
        return (0,)
    return SPECS[fam]
CHUNK = 6                                            # instances per translation unit


def _tile(c):
    bits, dk, dv, group, qbuf, mmax, axv = c
    return (f'Tile<{bits}, {dk}, {dv}, {group}, {"true" if qbuf else "false"}, {mmax}'
            + (', true>' if axv else '>'))


# Run-time conditions of the workgroup-per-key-head kernels, per family (part of the generated dispatch unit).
QUAD_OK = {'gdn': [
    '// q, k per key head (or ungrouped keys), rows that 16-byte vector loads can address',
    'static bool gdn_quad_ok(const GdnParams& p) {',
    '    if (!p.qk_per_key_head && p.gqa > 1) return false;',
    '    auto ok = [](const void* ptr, uint32_t stride, int dt) {',
    '        return reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && (uint64_t(stride) * (dt == 0 ? 4 : 2)) % 16 == 0;',
    '    };',
    '    return ok(p.q, p.s_q, p.q_dt) && ok(p.k, p.s_k, p.k_dt);',
    '}'],
    'mamba2': [
    '// B, C rows that 16-byte vector loads can address',
    'static bool mamba2_quad_ok(const Mamba2Params& p) {',
    '    auto ok = [](const void* ptr, uint32_t stride, int dt) {',
    '        return reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && (uint64_t(stride) * (dt == 0 ? 4 : 2)) % 16 == 0;',
    '    };',
    '    return ok(p.B, p.s_B, p.B_dt) && ok(p.C, p.s_C, p.C_dt);',
    '}']}


def quad_variants(fam, c):
    """[(row blocks per wavefront, value heads per workgroup, wavefronts per SIMD the register allocation aims
    for)], widest head group first, of the workgroup-per-key-head kernels (sq_quad.cuh) for a case; empty where only
    the one-wavefront kernels (sq_tile.cuh) serve it: value-axis groups, the float state, rows that are not a power
    of two in size, d_k above 128, more than four scale groups per row."""
    bits, dk, dv, group, qbuf, mmax, axv = c
    if fam not in QUAD_FAMILIES or axv or bits not in (4, 8):
        return []
    rb = dk * bits // 8
    if rb & (rb - 1) or not 32 <= rb <= 128 or dk > 128 or dv % 32 or (bits == 4 and dk % 64):
        return []
    if -(-dk // group) > 4:
        return []
    nrb = dv // 32
    nb = 2 if nrb % 2 == 0 else 1
    be = 1 if qbuf else 2
    out = []
    for gh in QUAD_FAMILIES[fam]:
        nw = gh * nrb // nb
        if nw > 16:
            continue
        lds = gh * dv * rb + mmax * dk * be + gh * mmax * dv * be + 2 * dk * 4 + dk * 8 + 512
        wgs = min(160 * 1024 // lds, 32 // nw)
        if wgs < 1:
            continue
        # register target: as many wavefronts per SIMD as LDS lets workgroups in, up to 6 (5 with the 16-token buffer);
        # asked for 7, the int4 kernels spill into scratch memory inside the fold (measured: +60 % bytes written)
        wpe = max(1, min(6 if mmax <= 8 else 5, -(-wgs * nw // 4)))
        # the serving cases compiled in (SPEC of the kernels) for the default buffer: int8, 8 tokens
        for spec in SPECS[fam] if (qbuf and mmax == 8) else (0,):
            out.append((nb, gh, wpe, spec))
    return out


def _quad_name(fam, c, v):
    nb, gh, wpe, spec = v
    return f'launch_{fam}_quad<{_tile(c)}, {nb}, {gh}, {wpe}, {spec}>'


def _write_if_changed(path, text):
    if os.path.exists(path) and open(path).read() == text:
        return
    with open(path, 'w') as f:
        f.write(text)


def generate():
    """Write the instance and dispatch translation units; returns their paths."""
    os.makedirs(OUT, exist_ok=True)
    units = []
    for fam, rows in CASES.items():
        insts = [(c, sp) for c in rows for sp in specs_of(fam, c, False)]
        for k in range(0, len(insts), CHUNK):
            body = ''.join(f'template int launch_{fam}<{_tile(c)}, {sp}>(const {PARAMS[fam]}&, hipStream_t);\n'
                           for c, sp in insts[k:k + CHUNK])
            path = os.path.join(OUT, f'inst_{fam}_{k // CHUNK:02d}.hip')
            _write_if_changed(path, f'// generated by build.py\n#include "../sq_{fam}.cuh"\nnamespace sq {{\n{body}}}\n')
            units.append(path)
    for fam, rows in CASES.items():
        qrows = [(c, v) for c in rows for v in quad_variants(fam, c)]
        for k in range(0, len(qrows), CHUNK):
            body = ''.join(f'template int {_quad_name(fam, c, v)}(const {PARAMS[fam]}&, hipStream_t);\n'
                           for c, v in qrows[k:k + CHUNK])
            path = os.path.join(OUT, f'inst_{fam}q_{k // CHUNK:02d}.hip')
            _write_if_changed(path, f'// generated by build.py\n#include "../sq_{fam}_quad.cuh"\nnamespace sq {{\n{body}}}\n')
            units.append(path)
    # pack / read: instances by (bits, d_k, group, value-axis[, buffer, per-channel decay]); d_v and m are run-time there
    rowfmt = sorted({(c[0], c[1], c[3], c[6]) for rows in CASES.values() for c in rows})
    kda_fmt = {(c[0], c[1], c[3], c[6]) for c in CASES['kda']}
    tf = lambda x: 'true' if x else 'false'                  # noqa: E731
    conv = [f'template int launch_pack<{b}, {dk}, {g}, {tf(v)}>(const PackParams&, hipStream_t);\n'
            for b, dk, g, v in rowfmt]
    reads = [(b, dk, g, v, q, k) for b, dk, g, v in rowfmt for q in (1, 0) for k in (0, 1)
             if not k or (b, dk, g, v) in kda_fmt]
    conv += [f'template int launch_read<{b}, {dk}, {g}, {tf(q)}, {tf(k)}, {tf(v)}>(const ReadParams&, hipStream_t);\n'
             for b, dk, g, v, q, k in reads]
    for k in range(0, len(conv), 2 * CHUNK):
        path = os.path.join(OUT, f'inst_convert_{k // (2 * CHUNK):02d}.hip')
        _write_if_changed(path, '// generated by build.py\n#include "../sq_convert.cuh"\nnamespace sq {\n'
                          + ''.join(conv[k:k + 2 * CHUNK]) + '}\n')
        units.append(path)
    path = os.path.join(OUT, 'inst_gga_00.hip')
    _write_if_changed(path, '// generated by build.py\n#include "../sq_gga.cuh"\nnamespace sq {\n'
                      + ''.join(f'template int launch_gga<GgaTile<{dk}, {dv}>>(const GgaParams&, int, hipStream_t);\n'
                                for dk, dv in GGA_SHAPES) + '}\n')
    units.append(path)
    d = ['// generated by build.py: layout -> compiled kernel instance', '#include <atomic>', '#include "../sq_convert.cuh"',
         'namespace sq {',
         '// Which instance serves a call when several could (results do not depend on it): set through sq_debug_select,',
         '// never read from the environment.',
         'static std::atomic<int> g_no_spec{0}, g_no_quad{0}, g_ghmax{64}, g_lds_pad{0};',
         'void select_instances(int no_spec, int no_quad, int ghmax, int lds_pad) {',
         '    g_no_spec.store(no_spec != 0);',
         '    g_no_quad.store(no_quad != 0);',
         '    g_ghmax.store(ghmax > 0 ? ghmax : 64);',
         '    g_lds_pad.store(lds_pad > 0 ? lds_pad : 0);',
         '}',
         'int quad_lds_pad() { return g_lds_pad.load(std::memory_order_relaxed); }']
    for fam, rows in CASES.items():
        P = PARAMS[fam]
        d.append(f'template <class T, int SPEC> int launch_{fam}(const {P}&, hipStream_t);')
        if fam in QUAD_FAMILIES:
            d.append(f'template <class T, int NB, int GH, int WPE, int SPEC> int launch_{fam}_quad(const {P}&, hipStream_t);')
            d += QUAD_OK[fam]
        d.append(f'int dispatch_{fam}(const {P}& p, hipStream_t stream, bool run) {{')
        d.append('    const int spec = (run && !g_no_spec.load(std::memory_order_relaxed)) ? serving_case(p) : 0;')
        if fam in QUAD_FAMILIES:
            d.append(f'    const bool quad = !g_no_quad.load(std::memory_order_relaxed) && (!run || {fam}_quad_ok(p));')
            d.append('    const int ghmax = g_ghmax.load(std::memory_order_relaxed);')
        # smallest sufficient buffer bound first
        for c in sorted(rows, key=lambda c: c[5]):
            bits, dk, dv, group, qbuf, mmax, axv = c
            cond = (f'p.bits == {bits} && p.dk == {dk} && p.dv == {dv} && p.group == {group} && p.axv == {axv} '
                    f'&& p.qbuf == {qbuf} && p.m <= {mmax}')
            for v in quad_variants(fam, c):
                want = f'spec == {v[3]} && ' if v[3] else ''             # the general instance takes whatever is left
                d.append(f'    if (quad && {want}p.gqa % {v[1]} == 0 && {v[1]} <= ghmax && {cond}) return run ? {_quad_name(fam, c, v)}(p, stream) : 0;')
            for sp in specs_of(fam, c, False):
                want = f'spec == {sp} && ' if sp else ''
                d.append(f'    if ({want}{cond}) return run ? launch_{fam}<{_tile(c)}, {sp}>(p, stream) : 0;')
        d.append('    return -1;\n}')
    d.append('template <int BITS, int DK, int GROUP, bool AXV> int launch_pack(const PackParams&, hipStream_t);')
    d.append('int dispatch_pack(const PackParams& p, hipStream_t stream, bool run) {')
    for b, dk, g, v in rowfmt:
        d.append(f'    if (p.bits == {b} && p.dk == {dk} && p.group == {g} && p.axv == {v}) '
                 f'return run ? launch_pack<{b}, {dk}, {g}, {tf(v)}>(p, stream) : 0;')
    d.append('    return -1;\n}')
    d.append('template <int BITS, int DK, int GROUP, bool QBUF, bool KDA, bool AXV> '
             'int launch_read(const ReadParams&, hipStream_t);')
    d.append('int dispatch_read(const ReadParams& p, hipStream_t stream, bool run) {')
    for b, dk, g, v, q, k in reads:
        d.append(f'    if (p.bits == {b} && p.dk == {dk} && p.group == {g} && p.axv == {v} && p.qbuf == {q} '
                 f'&& p.kda == {k}) return run ? '
                 f'launch_read<{b}, {dk}, {g}, {tf(q)}, {tf(k)}, {tf(v)}>(p, stream) : 0;')
    d.append('    return -1;\n}')
    d += ['int launch_fold_order(const int32_t* idx, const int32_t* NPTR, uint32_t sN, int m, int rows, int32_t* order,',
          '                      hipStream_t stream) {',
          '    hipLaunchKernelGGL((fold_order_kernel<FO_THREADS>), dim3(1), dim3(FO_THREADS), 0, stream, idx, NPTR, sN, m, rows, order);',
          '    return int(hipGetLastError());',
          '}']
    d.append('template <int DK, int DV> struct GgaTile;')
    d.append('template <class T> int launch_gga(const GgaParams&, int, hipStream_t);')
    d.append('int dispatch_gga(const GgaParams& p, int op, hipStream_t stream, bool run) {')
    for dk, dv in GGA_SHAPES:
        d.append(f'    if (p.dk == {dk} && p.dv == {dv} && p.m <= 8) '
                 f'return run ? launch_gga<GgaTile<{dk}, {dv}>>(p, op, stream) : 0;')
    d.append('    return -1;\n}')
    d.append('}  // namespace sq\n')
    path = os.path.join(OUT, 'dispatch.hip')
    _write_if_changed(path, '\n'.join(d))
    units.append(path)
    units.append(os.path.join(HERE, 'sq_api.hip'))
    return units


def _stamp():
    """Hash of every source that goes into the library (to skip a rebuild when nothing changed)."""
    h = hashlib.sha256()
    for name in sorted(os.listdir(HERE)):
        if name.endswith(('.cuh', '.h', '.hip', '.py')):
            h.update(open(os.path.join(HERE, name), 'rb').read())
    h.update(open(os.path.join(os.path.dirname(PKG), 'include', 'statequant_hip.h'), 'rb').read())
    h.update(' '.join(HIPCC_FLAGS).encode())
    return h.hexdigest()


_INCLUDE = re.compile(r'^\s*#\s*include\s+"([^"]+)"', re.M)


def _unit_hash(src, seen=None):
    """Hash of a translation unit with every header it includes by "quotes", transitively, and the flags."""
    seen = {} if seen is None else seen
    todo = [os.path.abspath(src)]
    while todo:
        path = todo.pop()
        if path in seen or not os.path.exists(path):
            continue
        text = open(path).read()
        seen[path] = text
        todo += [os.path.normpath(os.path.join(os.path.dirname(path), inc)) for inc in _INCLUDE.findall(text)]
    h = hashlib.sha256(' '.join(HIPCC_FLAGS).encode())
    for path in sorted(seen):
        h.update(path.encode())
        h.update(seen[path].encode())
    return h.hexdigest()


_SREG = re.compile(r'\bs(\d+)\b|\bs\[(\d+):(\d+)\]')


def lint_counter_loads(asm_text):
    """The workgroup kernels fetch a slot's fill counter with a scalar load written in assembly and wait for it in a
    second assembly statement further down (sq_quad.cuh: quad_dma_counter / quad_dma_counter_wait).  Between the two
    the destination register holds nothing yet, and the compiler -- which believes the value is there -- must not have
    read, copied or spilled it.  This walks the device assembly of a unit and returns one message per violation
    (empty list: fine)."""
    problems, pending, in_asm, func = [], None, False, '?'
    for no, line in enumerate(asm_text.split('\n'), 1):
        t = line.strip()
        if t.endswith(':') and not t.startswith(('.', ';')):
            func = t[:-1]
        if t.startswith(';;#ASMSTART'):
            in_asm = True
            continue
        if t.startswith(';;#ASMEND'):
            in_asm = False
            continue
        if not t or t[0] in '.;' or t.endswith(':'):
            continue
        if t.startswith('s_endpgm') and pending is not None:    # a path that leaves before the wait never uses it
            continue
        if in_asm:
            m = re.match(r's_load_dword s(\d+), ', t)
            if m:
                if pending is not None:
                    problems.append(f'{func}: line {no}: a second counter load before the wait for s{pending}')
                pending = int(m.group(1))
                continue
            if pending is not None and t.startswith('s_waitcnt') and 'lgkmcnt(0)' in t:
                pending = None
                continue
        if pending is None:
            continue
        code = t.split(';')[0]
        for m in _SREG.finditer(code):
            lo, hi = (int(m.group(1)),) * 2 if m.group(1) else (int(m.group(2)), int(m.group(3)))
            if lo <= pending <= hi:
                problems.append(f'{func}: line {no}: `{code.strip()}` touches s{pending} before its load is waited for')
                break
    if pending is not None:
        problems.append(f'{func}: counter load into s{pending} is never waited for')
    return problems


def _compile(src, force=False):
    """Compile one unit unless its object is current (same sources, headers and flags as when it was built).  Units of
    the workgroup kernels keep their device assembly long enough for lint_counter_loads to read it."""
    base = os.path.splitext(os.path.basename(src))[0]
    obj = os.path.join(OUT, base + '.o')
    tag, want = obj + '.hash', _unit_hash(src)
    if not force and os.path.exists(obj) and os.path.exists(tag) and open(tag).read() == want:
        return obj
    lint = base.startswith(tuple(f'inst_{fam}q_' for fam in QUAD_FAMILIES))
    cmd = ['hipcc', *HIPCC_FLAGS, *(['--save-temps=obj'] if lint else []), '-c', src, '-o', obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError(f'{" ".join(cmd)}\n{r.stdout}\n{r.stderr}')
    if lint:
        temps = [os.path.join(OUT, f) for f in os.listdir(OUT) if f.startswith(base + '-') or f.startswith(base + '.hip-')]
        asm = [f for f in temps if f.endswith(f'{ARCH}.s')]
        problems = lint_counter_loads(open(asm[0]).read()) if asm else [f'no device assembly kept for {src}']
        for f in temps:
            os.remove(f)
        if problems:
            os.remove(obj)
            raise RuntimeError(f'{src}: hand-placed scalar wait violated\n  ' + '\n  '.join(problems))
    with open(tag, 'w') as f:
        f.write(want)
    return obj


def build(jobs=None, force=False, verbose=True):
    """Compile and link; returns the path of the library."""
    jobs = jobs or min(16, os.cpu_count() or 4)
    units = generate()
    stamp_path = os.path.join(OUT, 'stamp')
    stamp = _stamp()
    if not force and os.path.exists(LIB) and os.path.exists(stamp_path) and open(stamp_path).read() == stamp:
        if verbose:
            print(f'[build] {LIB} is up to date')
        return LIB
    if verbose:
        n = sum(len(specs_of(fam, c, False)) + len(quad_variants(fam, c)) for fam, r in CASES.items() for c in r)
        print(f'[build] hipcc {ARCH}: {n} step-kernel instances in {len(units)} translation units, {jobs} jobs')
    with cf.ThreadPoolExecutor(jobs) as ex:
        objs = list(ex.map(lambda u: _compile(u, force), units))
    cmd = ['hipcc', '--offload-arch=' + ARCH, '-shared', '-fPIC', '-o', LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError(f'{" ".join(cmd)}\n{r.stdout}\n{r.stderr}')
    with open(stamp_path, 'w') as f:
        f.write(stamp)
    if verbose:
        print(f'[build] wrote {LIB} ({os.path.getsize(LIB) / 1e6:.1f} MB)')
    return LIB


_REMARK = re.compile(r'remark: +(Function Name|VGPRs|AGPRs|SGPRs Spill|VGPRs Spill|ScratchSize \[bytes/lane\]|'
                     r'Occupancy \[waves/SIMD\]|LDS Size \[bytes/block\]): +(\S+)')


def resources(pattern='', jobs=None):
    """Print one line per compiled kernel: what the compiler's -Rpass-analysis=kernel-resource-usage remarks state
    for it (device pass only, nothing is linked).  VGPRs and AGPRs share one file of 512 registers per SIMD lane."""
    jobs = jobs or min(16, os.cpu_count() or 4)
    units = [u for u in generate() if not u.endswith(('dispatch.hip', 'sq_api.hip'))]

    def one(src):
        cmd = ['hipcc', *HIPCC_FLAGS, '--cuda-device-only', '-Rpass-analysis=kernel-resource-usage', '-c', src,
               '-o', os.devnull]
        r = subprocess.run(cmd, capture_output=True, text=True)
        rows, cur = [], None
        for key, val in _REMARK.findall(r.stderr):
            if key == 'Function Name':
                cur = {'name': val}
                rows.append(cur)
            elif cur is not None:
                cur[key] = val
        return rows

    with cf.ThreadPoolExecutor(jobs) as ex:
        rows = [r for unit in ex.map(one, units) for r in unit]
    demangle = subprocess.run(['c++filt'], input='\n'.join(r['name'] for r in rows), capture_output=True, text=True)
    names = demangle.stdout.split('\n') if demangle.returncode == 0 else [r['name'] for r in rows]
    print('VGPR AGPR spill(V/S) scratch occupancy   LDS  kernel')
    for r, n in sorted(zip(rows, names), key=lambda x: x[1]):
        n = n.replace('sq::', '').replace('void ', '')
        n = n[:n.index('>(') + 1] if '>(' in n else n
        if pattern in n:
            print(f"{r.get('VGPRs', '?'):>4} {r.get('AGPRs', '?'):>4} {r.get('VGPRs Spill', '?'):>5}/{r.get('SGPRs Spill', '?'):<3} "
                  f"{r.get('ScratchSize [bytes/lane]', '?'):>6} {r.get('Occupancy [waves/SIMD]', '?'):>8} "
                  f"{r.get('LDS Size [bytes/block]', '?'):>6}  {n}")


if __name__ == '__main__':
    ap = argparse.ArgumentParser()
    ap.add_argument('-j', type=int, default=None)
    ap.add_argument('--force', action='store_true')
    ap.add_argument('--timeline', action='store_true',
                    help='build libsqhip_timeline.so instead: the same library with the workgroup-per-key-head Gated '
                         'DeltaNet kernel instrumented (-DSQ_TIMELINE, see sq_gdn_quad.cuh); profile_timeline.py '
                         'loads it.  Objects go to csrc/build_timeline/')
    ap.add_argument('--resources', metavar='PATTERN', nargs='?', const='', default=None,
                    help="instead of building, print the compiler's resource usage (registers, spills, LDS, "
                         'occupancy) of every kernel whose name contains PATTERN')
    a = ap.parse_args()
    if a.timeline:
        OUT = os.path.join(HERE, 'build_timeline')
        LIB = os.path.join(PKG, 'libsqhip_timeline.so')
        HIPCC_FLAGS = HIPCC_FLAGS + ['-DSQ_TIMELINE']
    if a.resources is not None:
        resources(a.resources, a.j)
        sys.exit(0)
    try:
        build(a.j, a.force)
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)
