"""Host-side logic that needs no GPU: storage format, per-slot byte layouts against the reference's documented
totals, the prefill-side read / write on CPU blobs, the C-ABI library's symbols, and loud failure off the GPU."""
import ctypes
import os
import re

import pytest
import torch

import statequant_amd as sq
from oracle import formats as F
from oracle import slots as OSL
from statequant_amd.kernels import (KDASlotLayout, Mamba2SlotLayout, PackedGDNState, SlotLayout, _hip, pack, pack_vk,
                                    packed_format, unpack, unpack_vk)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize('bits', [4, 8])
@pytest.mark.parametrize('axis', ['k', 'v'])
@pytest.mark.parametrize('group', [32, 64])
def test_pack_roundtrip_matches_fake(bits, axis, group):
    """unpack(pack(S)) == Quantizer(..., scale_dtype='fp16').fake(S) bit for bit, incl. all-zero groups and scales in
    the fp16 subnormal range (the reference's tests/test_kernels.py:26-49), and == the oracle's pack."""
    torch.manual_seed(0)
    S = torch.randn(8, 128, 128) * torch.rand(8, 128, 1) * 3
    S[0, :, :64] = 0
    S[1] *= 1e-6
    q = sq.Quantizer(bits, axis, group)
    codes, scales = pack(S, q)
    assert scales.dtype == torch.float16
    assert codes.dtype == (torch.uint8 if bits == 4 else torch.int8)
    assert codes.shape == (8, 128, 128 // (2 if bits == 4 else 1))
    got = unpack(codes, scales, q, 128)
    assert torch.equal(got, sq.Quantizer(bits, axis, group, scale_dtype='fp16').fake(S))
    assert torch.equal(packed_format(q).fake(S), got)
    oc, os_ = F.pack_vk(S.transpose(1, 2).contiguous(), (bits, axis, group))
    assert torch.equal(codes, oc) and torch.equal(scales, os_)
    c4, s4 = pack(S.reshape(2, 4, 128, 128), q)
    assert torch.equal(c4, codes) and torch.equal(s4, scales)
    # all-zero group: amax 1e-8 / qmax rounds to fp16 zero and is floored at 2^-24; codes 0
    if axis == 'k':
        assert (scales[0, :64].float() == 2.0 ** -24).all()          # S[0, :, :64] = 0: value rows 0..63 all zero


def test_ragged_key_group_and_bf16():
    X = torch.randn(3, 32, 96)
    q = sq.Quantizer(4, 'k', 64)
    c, s = pack_vk(X, q)
    assert s.shape == (3, 32, 2) and c.shape == (3, 32, 48)
    deq = unpack_vk(c, s, q, 96)
    # a ragged group is quantized on its own: same as quantizing the two column blocks separately
    a = unpack_vk(*pack_vk(X[..., :64].contiguous(), q), q, 64)
    b = unpack_vk(*pack_vk(X[..., 64:].contiguous(), sq.Quantizer(4, 'k', 32)), sq.Quantizer(4, 'k', 32), 32)
    assert torch.equal(deq, torch.cat([a, b], -1))
    S = torch.randn(4, 64, 64)
    cb, sb = pack(S, 'bf16')
    assert torch.equal(unpack(cb, sb, 'bf16', 64), S.to(torch.bfloat16).float())


def test_brute_force_per_group_numpy():
    """pack_vk against a scalar restatement with np.float16 on a tiny input (independent of torch's kernels)."""
    import numpy as np
    rng = np.random.default_rng(0)
    X = (rng.standard_normal((2, 4, 32)) * np.array([1.0, 1e-6])[:, None, None]).astype(np.float32)
    X[0, 1, :16] = 0
    for bits, g in ((4, 16), (8, 32)):
        qmax = 2 ** (bits - 1) - 1
        codes, scales = pack_vk(torch.from_numpy(X), sq.Quantizer(bits, 'k', g))
        deq = unpack_vk(codes, scales, sq.Quantizer(bits, 'k', g), 32).numpy()
        for n in range(2):
            for r in range(4):
                for gi in range(32 // g):
                    blk = X[n, r, gi * g:(gi + 1) * g]
                    s = np.float32(np.float16(np.float32(max(np.abs(blk).max(), np.float32(1e-8))) / np.float32(qmax)))
                    s = max(s, np.float32(2.0 ** -24))
                    want = np.clip(np.rint(blk / s), -qmax, qmax) * s
                    assert np.array_equal(deq[n, r, gi * g:(gi + 1) * g], want.astype(np.float32))


# per-slot bytes the reference documents for real models (docs/vllm.md:116-119, 143-146, 188-191 there)
DOC_TOTALS = [
    (SlotLayout, dict(hv=30, hk=30, dk=96, dv=192), {'pace4': 370816, 'int8k': 658816, 'int4v': 382336, 'bf16': 1177216}),
    (Mamba2SlotLayout, dict(hv=96, hk=8, dk=128, dv=80), {'pace4': 597376, 'int8k': 1119616, 'int4v16': 689536,
                                                           'bf16': 2041216}),
    (KDASlotLayout, dict(hv=16, dk=128, dv=128), {'pace4': 246336, 'int8k': 385600, 'int4v': 254528, 'bf16': 631360}),
]
PRESETS = {'pace4': sq.Quantizer(4, 'k', 64), 'int8k': sq.Quantizer(8, 'k', 32), 'int4v': sq.Quantizer(4, 'v', 32),
           'int4v16': sq.Quantizer(4, 'v', 16), 'bf16': 'bf16'}


def test_layout_bytes_match_documented_totals():
    for cls, shape, totals in DOC_TOTALS:
        for preset, nbytes in totals.items():
            lay = cls(PRESETS[preset], m=8, buffer_bits=8, **shape)
            assert lay.nbytes == nbytes, (cls.__name__, preset, lay.nbytes, nbytes)
            assert lay.nbytes == sum(-(-x // 16) * 16 for x in lay.breakdown().values())
    # the benchmark layouts: Qwen3.5-4B GDN, 32 value / 16 key heads, 128 x 128
    want = {(8, 32): 608256, (8, 128): 583680, (4, 64): 329728, (4, 32): 346112}
    for (bits, g), nbytes in want.items():
        lay = SlotLayout(sq.Quantizer(bits, 'k', g), 32, 16, 128, 128, m=8, buffer_bits=8)
        assert lay.nbytes == nbytes
    lay = SlotLayout(sq.Quantizer(4, 'k', 64), 32, 16, 128, 128, m=8, buffer_bits=8)
    b = lay.breakdown()                                            # the reference's tests/test_slots.py:210-216
    assert b['S'] == 32 * 128 * 64 and b['SC'] == 32 * 128 * 2 * 2 and b['KB'] == 16 * 8 * 128 and b['UB'] == 32 * 8 * 128
    assert KDASlotLayout(sq.Quantizer(4, 'k', 32), 32, 128, 128).nbytes == 509056
    assert list(lay.fields) == ['GB', 'GCUR', 'NPTR', 'SC', 'KBS', 'UBS', 'S', 'KB', 'UB']


@pytest.mark.parametrize('family', ['gdn', 'mamba2', 'kda'])
def test_layout_read_write_match_oracle(family):
    """Product layout == oracle layout, field by field; write / read on a CPU blob == the oracle's (torch code)."""
    fmt = (4, 'k', 32)
    if family == 'kda':
        lay = KDASlotLayout(sq.Quantizer(*fmt), 2, 32, 32, m=4, buffer_bits=8)
        hv, hk = 2, 2
    else:
        cls = SlotLayout if family == 'gdn' else Mamba2SlotLayout
        lay = cls(sq.Quantizer(*fmt), 4, 2, 32, 32, m=4, buffer_bits=8)
        hv, hk = 4, 2
    table, nbytes = OSL.layout(family, fmt, hv, hk, 32, 32, 4, 8)
    assert nbytes == lay.nbytes and table == lay.fields
    torch.manual_seed(1)
    blob = torch.randint(0, 256, (5, lay.nbytes), dtype=torch.uint8)
    blob2 = blob.clone()
    V, V2 = lay.views(blob), OSL.views(table, blob2)
    idx = torch.tensor([3, 1])
    S = torch.randn(2, hv, 32, 32)
    lay.write(V, idx, S)
    OSL.write(V2, idx, S, fmt, hv, 32, 32)
    assert torch.equal(blob, blob2)
    for W in (V, V2):
        W['NPTR'][idx] = 2
        W['GCUR'][idx] = -0.3
        W['GB'][idx] = -0.1
        W['KBS'][idx] = 0.01
        W['UBS'][idx] = 0.02
    got = lay.read(V, idx)
    want = OSL.read(V2, idx, fmt, hv, hk, 32, 32, 4, per_channel=family == 'kda')
    assert torch.allclose(got, want, rtol=1e-6, atol=1e-7)


def test_library_exports_every_declared_symbol():
    """libsqhip.so loads without a GPU and exports exactly the entry points include/statequant_hip.h declares."""
    header = open(os.path.join(ROOT, 'include', 'statequant_hip.h')).read()
    declared = set(re.findall(r'^\s*(?:int|void|const char\*)\s+(sq_\w+)\s*\(', header, flags=re.M))
    assert declared == set(_hip.SYMBOLS), declared ^ set(_hip.SYMBOLS)
    L = _hip.lib()
    for name in declared:
        assert hasattr(L, name), name
    assert L.sq_abi_version() == _hip.ABI_VERSION == 6
    assert L.sq_strerror(0) == b'ok'
    lay = _hip.SqLayout(bits=8, axis_k=1, group=128, buffer_bits=8, m=8, hv=32, hk=16, dk=128, dv=128)
    assert L.sq_supported(0, ctypes.byref(lay)) == 1
    lay.dv = 100
    assert L.sq_supported(0, ctypes.byref(lay)) == 0
    # argument errors are reported before anything touches a device
    assert L.sq_gdn_step(None, None) == -1 and b'null args' in L.sq_last_error()
    a = _hip.SqGdnArgs(lay=_hip.SqLayout(bits=5, axis_k=1, group=32, buffer_bits=8, m=8, hv=4, hk=2, dk=64, dv=64))
    assert L.sq_gdn_step(ctypes.byref(a), None) == -2 and b'bits' in L.sq_last_error()
    assert L.sq_fold_order(None, None, 0, 8, 64, None, None) == -1 and b'NPTR' in L.sq_last_error()
    assert L.sq_fold_order(None, None, 0, 8, 0, None, None) == 0               # no rows: nothing to do


def test_ctypes_structs_match_the_header():
    """Field order of the ctypes mirrors == the C structs (a reordering would silently shift every pointer)."""
    header = open(os.path.join(ROOT, 'include', 'statequant_hip.h')).read()
    for cname, S in (('sq_state', _hip.SqState), ('sq_layout', _hip.SqLayout), ('sq_gdn_args', _hip.SqGdnArgs),
                     ('sq_kda_args', _hip.SqKdaArgs), ('sq_mamba2_args', _hip.SqMamba2Args),
                     ('sq_pack_args', _hip.SqPackArgs), ('sq_read_args', _hip.SqReadArgs)):
        body = re.search(r'typedef struct %s \{(.*?)\} %s;' % (cname, cname), header, flags=re.S).group(1)
        body = re.sub(r'/\*.*?\*/', '', body, flags=re.S)
        names = []
        for decl in body.split(';'):
            decl = decl.strip()
            if decl:
                for part in decl.split(','):
                    names.append(re.findall(r'(\w+)\s*$', part.strip())[0])
        assert names == [f[0] for f in S._fields_], (cname, names)


def test_no_fallback_off_the_gpu():
    """CPU tensors never reach a kernel, and nothing else computes the step instead."""
    with pytest.raises(RuntimeError, match='GPU only'):
        PackedGDNState(torch.zeros(8, 64, 64), sq.Quantizer(4, 'k', 32), hv=4, hk=2)
    lay = SlotLayout(sq.Quantizer(4, 'v', 8), 4, 2, 128, 128)        # a layout with no kernel instance
    with pytest.raises(NotImplementedError):
        lay._layout_struct()
    SlotLayout(sq.Quantizer(4, 'v', 32), 4, 2, 128, 128)._layout_struct()


def test_bench_contract_off_the_gpu():
    """bench.py: more than one GPU is refused with a message (the step has no cross-GPU exchange to measure), and the
    byte model is the one the target is quoted on: (S + SC)(1 + 1/m) per slot and step."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, 'bench.py'), '--gpus', '2'], capture_output=True, text=True)
    assert r.returncode != 0 and 'one GPU' in r.stderr
    sys.path.insert(0, root)
    import bench
    per_slot = {'gdn-int8-g128': 599040, 'gdn-int8-g32': 626688, 'gdn-int4-g32': 331776, 'gdn-int4-g64': 313344,
                'mamba2-int8-g128': 1198080, 'kda-int4-g32': 331776, 'gdn-int4v-g32': 331776}
    for name, want in per_slot.items():
        fam, bits, group, hv, hk, dk, dv, slots, layers = bench.WORKLOADS[name]
        assert bench.state_bytes_per_slot(bits, group, hv, dk, dv, 8) == want, name
    assert bench.state_bytes_per_slot(8, 128, 32, 128, 128, 8) * 256 == 153354240


def test_timeline_marks_stay_out_of_the_product_library():
    """The timeline marks of the step kernels that carry them exist only behind -DSQ_TIMELINE: the default build
    never passes the define, `--timeline` builds a library and an object directory of their own, and the profiling
    script refuses to run without that library or without a GPU instead of falling back to anything."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    from statequant_amd.csrc import build
    assert '-DSQ_TIMELINE' not in build.HIPCC_FLAGS and build.LIB.endswith('libsqhip.so')
    src = open(os.path.join(root, 'statequant_amd', 'csrc', 'build.py')).read()
    assert "libsqhip_timeline.so" in src and "build_timeline" in src
    marks = open(os.path.join(root, 'statequant_amd', 'csrc', 'sq_timeline.cuh')).read()
    assert marks.count('#ifdef SQ_TIMELINE') == 1 and '#define SQ_MARK(k) do { } while (0)' in marks
    for name in ('sq_gdn_quad.cuh', 'sq_kda.cuh'):                     # the marked kernels
        kern = open(os.path.join(root, 'statequant_amd', 'csrc', name)).read()
        assert '#include "sq_timeline.cuh"' in kern and 'SQ_MARK(0)' in kern and '#ifdef SQ_TIMELINE' in kern
    if not torch.cuda.is_available():
        r = subprocess.run([sys.executable, os.path.join(root, 'profile_timeline.py')], capture_output=True, text=True)
        assert r.returncode != 0 and ('is missing' in r.stderr or 'no GPU visible' in r.stderr), r.stderr
    # the marked kernel still compiles (device pass of one instance, nothing linked)
    import shutil
    import tempfile
    if shutil.which('hipcc'):
        with tempfile.TemporaryDirectory() as d:
            unit = os.path.join(d, 'one.hip')
            with open(unit, 'w') as f:
                csrc = os.path.join(root, 'statequant_amd', 'csrc')
                f.write('#include "%s"\n#include "%s"\nnamespace sq {\n'
                        'template int launch_gdn_quad<Tile<8, 128, 128, 128, true, 8>, 2, 2, 4, 1>(const GdnParams&, '
                        'hipStream_t);\n'
                        'template int launch_kda<Tile<4, 128, 128, 32, true, 8>, 1>(const KdaParams&, hipStream_t);\n}\n'
                        % (os.path.join(csrc, 'sq_gdn_quad.cuh'), os.path.join(csrc, 'sq_kda.cuh')))
            r = subprocess.run(['hipcc', *build.HIPCC_FLAGS, '-DSQ_TIMELINE', '--cuda-device-only', '-c', unit, '-o',
                                os.path.join(d, 'one.o')], capture_output=True, text=True)
            assert r.returncode == 0, r.stderr[-2000:]


def test_gga_packed_tables_match_the_reference(golden):
    """``GGAPacked``: per-layer offset tables, window placement, slot size and bits per value as the reference's class
    computes them for the plan of its own tests (recorded in tests/golden/gga.pt); no GPU, no library call."""
    from statequant_amd.kernels.gga import GGAPacked, GGAPlan, head_bytes
    t = golden('gga.pt')['tables']
    hv, dk, dv, m = t['hv'], t['dk'], t['dv'], t['m']
    plan = GGAPlan({i: (torch.tensor(wd), torch.ones(hv, dk)) for i, wd in enumerate(t['widths'])})
    for pw in (False, True):
        pk = GGAPacked(plan, hv, 4, dk, dv, pw=pw, m=m)
        ref = t[pw]
        assert [pk.tables[i][0] for i in range(2)] == ref['offs']
        assert [pk.bytes_per_layer[i] for i in range(2)] == ref['bytes_per_layer']
        assert (pk.QOFF, pk.QSZ, pk.nbytes) == (ref['QOFF'], ref['QSZ'], ref['nbytes'])
        assert abs(pk.bits_per_value() - ref['bits_per_value']) < 1e-12
        blob = torch.zeros(3, pk.nbytes + 16, dtype=torch.uint8)
        assert pk.views(blob)['blob'] is blob
    assert [head_bytes(b, 128, 128) for b in (2, 4, 6, 8, 16)] == [5376, 8704, 12800, 16896, 32768]
    with pytest.raises(AssertionError):
        GGAPacked(GGAPlan({0: (torch.tensor([3] * hv), torch.ones(hv, dk))}), hv, 4, dk, dv)     # no 3-bit heads
    with pytest.raises(RuntimeError, match='GPU only'):
        pk.stored(pk.views(blob), torch.tensor([1]), 0)                                          # CPU blob: loud


def test_gga_bench_byte_model():
    import sys
    sys.path.insert(0, ROOT)
    import bench
    from statequant_amd.kernels.gga import GGAPacked
    pk = GGAPacked(bench.gga_plan(32, 128, 2), 32, 16, 128, 128, pw=True, m=8)
    state = 12 * 5376 + 11 * 8704 + 6 * 12800 + 2 * 16896 + 32768
    window = 31 * (8 * (128 + 128 + 8) + 8 * (128 + 4) + 128 + 128 + 8)
    assert bench.gga_bytes_per_slot_step(pk, 0) == 2 * state + window == 713624


def test_ctypes_structs_match_the_c_header(tmp_path):
    """Every argument struct of include/statequant_hip.h as gcc lays it out (size and the offset of each field)
    against its ctypes mirror in statequant_amd/kernels/_hip.py: a field added, dropped or retyped on one side only
    would shift everything behind it."""
    import subprocess
    pairs = {'sq_state': _hip.SqState, 'sq_layout': _hip.SqLayout, 'sq_gdn_args': _hip.SqGdnArgs,
             'sq_kda_args': _hip.SqKdaArgs, 'sq_mamba2_args': _hip.SqMamba2Args, 'sq_pack_args': _hip.SqPackArgs,
             'sq_read_args': _hip.SqReadArgs, 'sq_gga_slots': _hip.SqGgaSlots, 'sq_gga_args': _hip.SqGgaArgs}
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{os.path.join(ROOT, "include", "statequant_hip.h")}"',
             'int main(void) {']
    for cname, T in pairs.items():
        lines.append(f'  printf("{cname} %zu", sizeof({cname}));')
        for fname, _ in T._fields_:
            lines.append(f'  printf(" %zu", offsetof({cname}, {fname}));')
        lines.append('  printf("\\n");')
    lines += ['  return 0;', '}']
    src, exe = tmp_path / 'abi.c', tmp_path / 'abi'
    src.write_text('\n'.join(lines))
    subprocess.run(['gcc', '-std=c11', '-o', str(exe), str(src)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.strip().split('\n')
    assert len(out) == len(pairs)
    for line in out:
        name, size, *offs = line.split()
        T = pairs[name]
        assert int(size) == ctypes.sizeof(T), name
        assert [int(o) for o in offs] == [getattr(T, f).offset for f, _ in T._fields_], name


def test_unsupported_dims_refused_and_olmo_bytes():
    """The constructor's refusals and the OLMo-Hybrid-7B byte counts (tests/test_kernels_nonpow2.py:308-321 there)."""
    with pytest.raises(AssertionError, match='value group'):
        SlotLayout(sq.Quantizer(4, 'v', 128), 4, 2, 96, 192)
    with pytest.raises(AssertionError, match='multiple of 32'):
        SlotLayout('bf16', 4, 2, 96, 80)
    b = SlotLayout(sq.Quantizer(4, 'k', 64), 30, 30, 96, 192, m=8, buffer_bits=8).breakdown()
    assert b['S'] == 30 * 192 * 48 and b['SC'] == 30 * 192 * 2 * 2
    assert b['KB'] == 30 * 8 * 96 and b['UB'] == 30 * 8 * 192
    from statequant_amd.kernels import Mamba2SlotLayout
    assert Mamba2SlotLayout('bf16', 96, 8, 128, 80, m=8, buffer_bits=8).breakdown()['S'] == 96 * 80 * 128 * 2


def test_host_tensors_are_refused_before_any_launch():
    """Every wrapper that hands raw pointers to the library checks devices first: with CPU tensors the call ends in a
    RuntimeError raised in Python, not in a kernel dereferencing a host pointer."""
    from statequant_amd.kernels.gga import GGAPacked, GGAPlan
    B, HV, HK, D, m = 2, 4, 2, 128, 4
    idx = torch.tensor([1, 2], dtype=torch.int32)
    q, k, v = torch.zeros(B, HK, D), torch.zeros(B, HK, D), torch.zeros(B, HV, D)
    out = torch.zeros(B, HV, D)
    lay = SlotLayout(sq.Quantizer(8, 'k', 128), HV, HK, D, D, m=m)
    with pytest.raises(RuntimeError, match='GPU only'):
        lay.step(lay.views(lay.alloc(3, 'cpu')), idx, q, k, v, out, 1.0, g=torch.zeros(B, HV), beta=torch.zeros(B, HV))
    kl = KDASlotLayout(sq.Quantizer(4, 'k', 32), HV, D, D, m=m)
    with pytest.raises(RuntimeError, match='GPU only'):
        kl.step(kl.views(kl.alloc(3, 'cpu')), idx, torch.zeros(B, HV, D), torch.zeros(B, HV, D), v,
                torch.zeros(B, HV, D), torch.zeros(B, HV), out)
    ml = Mamba2SlotLayout(sq.Quantizer(8, 'k', 128), HV, HK, D, 64, m=m)
    with pytest.raises(RuntimeError, match='GPU only'):
        ml.step(ml.views(ml.alloc(3, 'cpu')), idx, torch.zeros(B, HV, 64), torch.zeros(B, HV), q, k,
                torch.zeros(B, HV, 64), torch.zeros(HV))
    pk = GGAPacked(GGAPlan({0: (torch.tensor([4] * HV), torch.ones(HV, D))}), HV, HK, D, D, pw=True)
    with pytest.raises(RuntimeError, match='GPU only'):
        pk.write(pk.views(pk.alloc(3, 'cpu')), idx, torch.zeros(B, HV, D, D), layer=0)
    # the helper itself: a state on one device and an operand on another
    class On:                                              # stands in for tensors on two GPUs
        def __init__(self, d):
            self.is_cuda, self.device = True, d
    with pytest.raises(RuntimeError, match='`idx` is on cpu'):
        _hip.same_device('step', On('cuda:0'), q=On('cuda:0'), idx=torch.zeros(1), beta=None)
    _hip.same_device('step', On('cuda:0'), q=On('cuda:0'), beta=None)


def test_gga_window_selects_dead_entries_away():
    """`GGAPacked.window` on a slot whose page was never zero-filled: dead ring entries decode to NaN (FP8 0xFF) with
    NaN scales and must come back as zeros, as the reference's `where(live, ..., 0)` gives them
    (vllm_gga.py, window()); live entries are untouched by the garbage around them."""
    from statequant_amd.kernels.gga import GGAPacked, GGAPlan
    HV, HK, D, m = 4, 2, 64, 4
    pk = GGAPacked(GGAPlan({0: (torch.tensor([4, 8, 16, 2]), torch.ones(HV, D))}), HV, HK, D, D, pw=True, m=m)
    blob = torch.full((3, pk.alloc(1, 'cpu').shape[1]), 0xFF, dtype=torch.uint8)
    views = pk.views(blob)
    idx = torch.tensor([1, 2])
    blob[:, :8] = 0                                        # counters: empty windows
    left, right, count = pk.window(views, idx)
    assert count.tolist() == [0, 0]
    assert torch.equal(left, torch.zeros_like(left)) and torch.equal(right, torch.zeros_like(right))
    # two live entries in slot 2 (ring positions 3 and 0), the other two entries garbage
    blob[2, :8] = torch.tensor([2, 3], dtype=torch.int32).view(torch.uint8)
    win = blob[2, pk.QOFF:pk.QOFF + HV * pk.QSZ].view(HV, pk.QSZ)
    one = torch.tensor([1.0], dtype=torch.float32).to(torch.float8_e4m3fn).view(torch.uint8).item()
    for pos in (3, 0):
        win[:, pos * D:(pos + 1) * D] = one                                           # left codes: all 1.0
        win[:, m * D + pos * D:m * D + (pos + 1) * D] = one                           # right codes
    sc = win[:, m * 2 * D:].view(torch.float32).view(HV, 2, m)
    sc[:, :, 3], sc[:, :, 0] = 0.5, 2.0
    left, right, count = pk.window(views, idx)
    assert count.tolist() == [0, 2]
    assert torch.isfinite(left).all() and torch.isfinite(right).all()
    assert torch.equal(left[1, 0], torch.full((HV, D), 0.5)) and torch.equal(left[1, 1], torch.full((HV, D), 2.0))
    assert torch.equal(left[1, 2:], torch.zeros(2, HV, D)) and torch.equal(left[0], torch.zeros(m, HV, D))


def test_build_lint_of_the_hand_placed_scalar_wait():
    """build.py reads the device assembly of every workgroup-kernel unit and refuses a build in which the register of
    the fill counter's scalar load (requested in one assembly statement, waited for in another) is touched in
    between: here the checker itself, on assembly with and without such a violation."""
    from statequant_amd.csrc.build import lint_counter_loads
    good = '\n'.join(['_Zkernel:', '\ts_mov_b32 s3, 0', '\t;;#ASMSTART', '\ts_load_dword s14, s[8:9], 0x0', '\t;;#ASMEND',
                      '\tv_mov_b32 v1, s15', '\ts_add_u32 s16, s12, s13', '\t;;#ASMSTART', '\ts_waitcnt lgkmcnt(0)',
                      '\t;;#ASMEND', '\ts_and_b32 s14, s14, 7', '\ts_endpgm'])
    assert lint_counter_loads(good) == []
    copied = good.replace('v_mov_b32 v1, s15', 's_mov_b32 s20, s14')
    assert len(lint_counter_loads(copied)) == 1 and 's_mov_b32 s20, s14' in lint_counter_loads(copied)[0]
    in_range = good.replace('s_add_u32 s16, s12, s13', 's_load_dwordx4 s[12:15], s[0:1], 0x0')
    assert len(lint_counter_loads(in_range)) == 1
    no_wait = good.replace('\t;;#ASMSTART\n\ts_waitcnt lgkmcnt(0)\n\t;;#ASMEND\n', '')
    assert any('never waited for' in m for m in lint_counter_loads(no_wait))
    # a compiler-placed wait does not count: only the assembly statement's own does
    compiler_wait = good.replace('\t;;#ASMSTART\n\ts_waitcnt lgkmcnt(0)\n\t;;#ASMEND\n', '\ts_waitcnt lgkmcnt(0)\n')
    assert lint_counter_loads(compiler_wait) != []
