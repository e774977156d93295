"""ctypes binding of libsqhip.so (the C ABI declared in ``include/statequant_hip.h``).

The library is built in-tree by ``python -m statequant_amd.csrc.build`` and must be present: there is no fallback
path.  ``lib()`` raises ``RuntimeError`` when it is missing, so a decode step can never silently run anywhere but in
the HIP kernels.
"""
from __future__ import annotations

import ctypes as C
import os

import torch

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG, 'libsqhip.so')
ABI_VERSION = 6

F32, BF16, F16 = 0, 1, 2
_DT = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
FAMILY = {'gdn': 0, 'kda': 1, 'mamba2': 2}

SYMBOLS = ('sq_abi_version', 'sq_strerror', 'sq_last_error', 'sq_supported', 'sq_gdn_step', 'sq_kda_step',
           'sq_mamba2_step', 'sq_pack_vk', 'sq_read', 'sq_fold_order', 'sq_debug_select', 'sq_gga_step', 'sq_gga_store', 'sq_gga_load',
           'sq_gga_supported')
E_UNSUPPORTED = -2

_vp, _i32, _i64, _f32 = C.c_void_p, C.c_int32, C.c_int64, C.c_float


class SqState(C.Structure):
    _fields_ = [('S', _vp), ('sS', _i64), ('SC', _vp), ('sSC', _i64), ('KB', _vp), ('sKB', _i64),
                ('KBS', _vp), ('sKBS', _i64), ('UB', _vp), ('sUB', _i64), ('UBS', _vp), ('sUBS', _i64),
                ('GB', _vp), ('sGB', _i64), ('GCUR', _vp), ('sGC', _i64), ('NPTR', _vp), ('sN', _i64)]


class SqLayout(C.Structure):
    _fields_ = [('bits', _i32), ('axis_k', _i32), ('group', _i32), ('buffer_bits', _i32), ('m', _i32),
                ('hv', _i32), ('hk', _i32), ('dk', _i32), ('dv', _i32)]


class SqGdnArgs(C.Structure):
    _fields_ = [('st', SqState), ('lay', SqLayout), ('rows', _i32), ('idx', _vp),
                ('q', _vp), ('s_q', _i64), ('q_dtype', _i32),
                ('k', _vp), ('s_k', _i64), ('k_dtype', _i32),
                ('v', _vp), ('s_v', _i64), ('v_dtype', _i32),
                ('qk_per_key_head', _i32), ('gate', _i32),
                ('g', _vp), ('s_g', _i64), ('g_dtype', _i32),
                ('beta', _vp), ('s_beta', _i64), ('beta_dtype', _i32),
                ('a', _vp), ('s_a', _i64), ('a_dtype', _i32),
                ('b', _vp), ('s_b', _i64), ('b_dtype', _i32),
                ('A_log', _vp), ('A_log_dtype', _i32),
                ('dt_bias', _vp), ('dt_bias_dtype', _i32),
                ('out', _vp), ('out_dtype', _i32), ('scale', _f32), ('order', _vp)]


class SqKdaArgs(C.Structure):
    _fields_ = [('st', SqState), ('lay', SqLayout), ('rows', _i32), ('idx', _vp),
                ('q', _vp), ('s_q', _i64), ('q_dtype', _i32),
                ('k', _vp), ('s_k', _i64), ('k_dtype', _i32),
                ('v', _vp), ('s_v', _i64), ('v_dtype', _i32),
                ('g', _vp), ('s_g', _i64), ('g_dtype', _i32),
                ('beta', _vp), ('s_beta', _i64), ('beta_dtype', _i32),
                ('out', _vp), ('s_out', _i64), ('out_dtype', _i32), ('scale', _f32), ('order', _vp)]


class SqMamba2Args(C.Structure):
    _fields_ = [('st', SqState), ('lay', SqLayout), ('rows', _i32), ('idx', _vp),
                ('x', _vp), ('s_x', _i64), ('x_dtype', _i32),
                ('dt', _vp), ('s_dt', _i64), ('dt_dtype', _i32),
                ('B', _vp), ('s_B', _i64), ('B_dtype', _i32),
                ('C', _vp), ('s_C', _i64), ('C_dtype', _i32),
                ('A', _vp), ('A_dtype', _i32), ('D', _vp), ('D_dtype', _i32),
                ('dt_bias', _vp), ('dt_bias_dtype', _i32),
                ('dt_softplus', _i32), ('dt_clamp', _i32), ('dt_min', _f32), ('dt_max', _f32),
                ('out', _vp), ('s_out', _i64), ('out_dtype', _i32), ('order', _vp)]


class SqPackArgs(C.Structure):
    _fields_ = [('lay', SqLayout), ('rows', _i32), ('idx', _vp), ('src', _vp), ('s_src', _i64),
                ('S', _vp), ('sS', _i64), ('SC', _vp), ('sSC', _i64),
                ('GCUR', _vp), ('sGC', _i64), ('gcur_per_head', _i32), ('NPTR', _vp), ('sN', _i64), ('nptr_copies', _i32)]


class SqReadArgs(C.Structure):
    _fields_ = [('st', SqState), ('lay', SqLayout), ('kda', _i32), ('rows', _i32), ('idx', _vp),
                ('out', _vp), ('s_out', _i64)]


class SqGgaSlots(C.Structure):
    _fields_ = [('blob', _vp), ('slot_stride', _i64), ('offs', _vp), ('bits', _vp), ('w', _vp),
                ('hv', _i32), ('hk', _i32), ('dk', _i32), ('dv', _i32), ('m', _i32), ('pw', _i32),
                ('qoff', _i64), ('qsz', _i64)]


class SqGgaArgs(C.Structure):
    _fields_ = [('sl', SqGgaSlots), ('rows', _i32), ('idx', _vp),
                ('q', _vp), ('s_q', _i64), ('q_dtype', _i32),
                ('k', _vp), ('s_k', _i64), ('k_dtype', _i32),
                ('v', _vp), ('s_v', _i64), ('v_dtype', _i32),
                ('gate', _i32),
                ('g', _vp), ('s_g', _i64), ('g_dtype', _i32),
                ('beta', _vp), ('s_beta', _i64), ('beta_dtype', _i32),
                ('a', _vp), ('s_a', _i64), ('a_dtype', _i32),
                ('b', _vp), ('s_b', _i64), ('b_dtype', _i32),
                ('A_log', _vp), ('A_log_dtype', _i32),
                ('dt_bias', _vp), ('dt_bias_dtype', _i32),
                ('out', _vp), ('out_dtype', _i32), ('scale', _f32)]


_lib = None


def lib():
    """The loaded library; raises if it has not been built or does not match this binding."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f'{LIB_PATH} is missing: build it with `python -m statequant_amd.csrc.build` '
                               '(the packed decode step has no fallback path)')
        L = C.CDLL(LIB_PATH)
        L.sq_abi_version.restype = C.c_int
        L.sq_strerror.restype = C.c_char_p
        L.sq_strerror.argtypes = [C.c_int]
        L.sq_last_error.restype = C.c_char_p
        L.sq_supported.restype = C.c_int
        L.sq_supported.argtypes = [C.c_int, C.POINTER(SqLayout)]
        for name, T in (('sq_gdn_step', SqGdnArgs), ('sq_kda_step', SqKdaArgs), ('sq_mamba2_step', SqMamba2Args),
                        ('sq_pack_vk', SqPackArgs), ('sq_read', SqReadArgs)):
            f = getattr(L, name)
            f.restype = C.c_int
            f.argtypes = [C.POINTER(T), C.c_void_p]
        L.sq_gga_step.restype = C.c_int
        L.sq_gga_step.argtypes = [C.POINTER(SqGgaArgs), C.c_void_p]
        for name in ('sq_gga_store', 'sq_gga_load'):
            f = getattr(L, name)
            f.restype = C.c_int
            f.argtypes = [C.POINTER(SqGgaSlots), C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p]
        L.sq_fold_order.restype = C.c_int
        L.sq_fold_order.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
        L.sq_debug_select.restype = None
        L.sq_debug_select.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32]
        L.sq_gga_supported.restype = C.c_int
        L.sq_gga_supported.argtypes = [C.c_int32, C.c_int32, C.c_int32]
        if L.sq_abi_version() != ABI_VERSION:
            raise RuntimeError(f'{LIB_PATH}: ABI version {L.sq_abi_version()}, this package expects {ABI_VERSION}')
        _lib = L
    return _lib


def dtype_code(t):
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f'float tensor of dtype fp32 / bf16 / fp16 expected, got {t.dtype}') from None


def ptr(t):
    return None if t is None else t.data_ptr()


def make_layout(st):
    """``SqLayout`` from a layout / state object with the reference's attribute names (bits, axk, group, ...)."""
    bits = st.bits                                        # 16: the unquantized state, bf16 -- or fp32 (slot layouts)
    if st.fmt is None and getattr(st, 'state_dtype', None) == torch.float32:
        bits = 32
    return SqLayout(bits=bits, axis_k=int(st.axk), group=st.group, buffer_bits=st.buffer_bits, m=st.m,
                    hv=st.HV, hk=st.HK, dk=st.DK, dv=st.DV)


def supported(family, st):
    lay = make_layout(st)
    return bool(lib().sq_supported(FAMILY[family], C.byref(lay)))


def make_state(T, strides, nptr_stride):
    """``SqState`` from the nine state tensors (dict) and their per-sequence strides in elements."""
    sS, sSC, sKB, sKBS, sUB, sUBS, sGB, sGC = strides
    return SqState(S=ptr(T['S']), sS=sS, SC=ptr(T['SC']), sSC=sSC, KB=ptr(T['KB']), sKB=sKB,
                   KBS=ptr(T['KBS']), sKBS=sKBS, UB=ptr(T['UB']), sUB=sUB, UBS=ptr(T['UBS']), sUBS=sUBS,
                   GB=ptr(T['GB']), sGB=sGB, GCUR=ptr(T['GCUR']), sGC=sGC, NPTR=ptr(T['NPTR']), sN=nptr_stride)


def current_stream(device):
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def check(rc):
    if rc != 0:
        L = lib()
        raise RuntimeError(f'libsqhip: {L.sq_strerror(rc).decode()}: {L.sq_last_error().decode()}')


def pack_into(lay, src, S, sS, SC, sSC, idx=None, GCUR=None, sGC=0, gcur_per_head=1, NPTR=None, sN=0):
    """``sq_pack_vk``: fp32 value-major ``src`` [rows, hv, dv, dk] (contiguous) -> codes ``S`` / scales ``SC`` (None
    for an unquantized state, which is cast) of the sequences ``idx`` (int32; None: sequence b), optionally emptying
    their buffers.  Raises when the library has no instance for the format, like every other error: GPU tensors never
    take another path."""
    assert src.dtype == torch.float32 and src.is_contiguous()
    rows = src.shape[0]
    a = SqPackArgs(lay=lay, rows=rows, idx=ptr(idx), src=src.data_ptr(), s_src=src.stride(0) if rows else 0,
                   S=S.data_ptr(), sS=sS, SC=ptr(SC), sSC=sSC, GCUR=ptr(GCUR), sGC=sGC,
                   gcur_per_head=gcur_per_head, NPTR=ptr(NPTR), sN=sN,
                   nptr_copies=0 if NPTR is None else NPTR[0].numel())
    check(lib().sq_pack_vk(C.byref(a), current_stream(src.device)))


def read_state(lay, T, strides, nptr_stride, idx, out, kda):
    """``sq_read``: the current state of sequences ``idx`` (int32) into fp32 ``out`` [rows, hv, dv, dk] (contiguous);
    rows with ``idx <= 0`` come back as zeros.  Raises when the library has no instance for the layout."""
    assert out.dtype == torch.float32 and out.is_contiguous()
    rows = out.shape[0]
    a = SqReadArgs(st=make_state(T, strides, nptr_stride), lay=lay, kda=int(kda), rows=rows, idx=ptr(idx),
                   out=out.data_ptr(), s_out=out.stride(0) if rows else 0)
    check(lib().sq_read(C.byref(a), current_stream(out.device)))


def fold_order(NPTR, nptr_stride, m, idx, out=None):
    """``sq_fold_order``: a dispatch order for the step calls' ``order`` argument (int32 [rows], on the device) from
    the fill counters ``NPTR`` (per-sequence stride ``nptr_stride`` in elements) of the sequences ``idx`` (int32
    [rows]; None: sequence b): the rows that fold on the coming step dealt evenly over the launch, the others in batch
    order.  ``out``: where to write it (no allocation then: graph-capturable).  Results of a step never depend on
    its order; with sequences out of step it shortens the launch.  No counterpart in the reference."""
    rows = idx.shape[0] if idx is not None else NPTR.shape[0]
    same_device('fold_order', NPTR, idx=idx, out=out)
    assert NPTR.dtype == torch.int32 and (idx is None or (idx.dtype == torch.int32 and idx.is_contiguous()))
    if out is None:
        out = torch.empty(rows, dtype=torch.int32, device=NPTR.device)
    assert out.dtype == torch.int32 and out.is_contiguous() and out.shape[0] >= rows
    check(lib().sq_fold_order(ptr(idx), NPTR.data_ptr(), nptr_stride, m, rows, out.data_ptr(),
                              current_stream(NPTR.device)))
    return out


def check_order(order, rows, ref):
    """The step wrappers' check of an ``order`` argument (None passes)."""
    if order is not None:
        assert order.dtype == torch.int32 and order.is_contiguous() and order.shape[0] >= rows
        same_device('step', ref, order=order)
    return ptr(order)


def select_instances(no_specialised=False, no_group_kernel=False, max_heads_per_workgroup=0, lds_pad_bytes=0):
    """``sq_debug_select``: which compiled instance serves a step call when several can (a diagnostic for twin tests
    and profiles; results do not depend on it).  ``lds_pad_bytes`` adds unused dynamic LDS to the workgroup kernels'
    launches (fewer resident workgroups).  Call without arguments to restore the default choice."""
    lib().sq_debug_select(int(no_specialised), int(no_group_kernel), int(max_heads_per_workgroup), int(lds_pad_bytes))


def require_gpu(t, what):
    if not t.is_cuda:
        raise RuntimeError(f'{what}: the packed decode step runs on the GPU only (HIP kernels, no fallback); '
                           f'got a tensor on {t.device}')


def same_device(what, ref, **tensors):
    """Raise unless ``ref`` is on a GPU and every given tensor (None: skipped) is on that same device.  The kernels
    receive raw pointers: a host tensor among them would be a GPU memory fault, not a Python error, so every wrapper
    calls this before it takes a pointer."""
    require_gpu(ref, what)
    for name, t in tensors.items():
        if t is not None and t.device != ref.device:
            raise RuntimeError(f'{what}: `{name}` is on {t.device}, the state on {ref.device}')
