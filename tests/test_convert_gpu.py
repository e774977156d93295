"""The HIP pack (`sq_pack_vk`: ``pack_vk`` / ``SlotLayout.write``) and read (`sq_read`: ``SlotLayout.read``) kernels
against the CPU oracle.  pack / write: bit-exact (same IEEE divisions and rounding as the reference's torch code,
fold.py:123-147, slots.py:236-252).  read: fp32 sums in another order than torch's einsum -> 1e-5 relative.
Formats: key-axis groups, value-axis groups of 32 rows, and the unquantized bf16 / fp32 state.
"""
import pytest
import torch

import statequant_amd as sq
from oracle import formats as OF
from oracle import slots as OS
from statequant_amd.kernels import KDASlotLayout, Mamba2SlotLayout, SlotLayout, pack_vk
from tests._util import gdn_token, quantizer
from tests.test_kda_gpu import kda_token
from tests.test_mamba2_gpu import m2_token, params

pytestmark = pytest.mark.gpu
DEV = 'cuda'


@pytest.mark.parametrize('fmt', [(8, 'k', 128), (8, 'k', 32), (4, 'k', 64), (4, 'k', 32), (8, 'v', 32), (4, 'v', 32), (8, 'v', 64),
                                 (4, 'v', 64), (8, 'v', 16), (4, 'v', 16)])
@pytest.mark.parametrize('dv,dk', [(128, 128), (64, 64), (192, 96), (96, 96)])
def test_pack_matches_oracle(fmt, dv, dk):
    if fmt[1] == 'k' and fmt[2] > (1 << (dk - 1).bit_length()):
        pytest.skip('group longer than the padded row')
    if fmt[1] == 'v' and (dv % fmt[2] or (fmt[2] == 16 and dk == 96)):
        pytest.skip('value-axis group does not divide d_v / not built for this d_k')
    gen = torch.Generator().manual_seed(dv + dk + fmt[0] + fmt[2])
    x = torch.randn(37, dv, dk, generator=gen)
    x[0] = 0.0                                             # all-zero heads: scale floor, codes 0
    x[1, :, : dk // 2] = 0.0                               # zero groups next to live ones
    x[2] *= 1e-6                                           # scales in the fp16 subnormal range
    x[3] *= 1e4
    x[4, 5] = 65504.0 * 127                                # scale at the top of fp16
    x[5, :32, 7] = 0.0                                     # value-axis: an all-zero group next to live ones
    codes, sc = pack_vk(x.to(DEV), quantizer(fmt))
    want_c, want_s = OF.pack_vk(x, fmt)
    assert codes.dtype == want_c.dtype and codes.shape == want_c.shape and sc.shape == want_s.shape
    assert torch.equal(sc.cpu(), want_s)
    assert torch.equal(codes.cpu(), want_c)


def _blob_pair(lay, table_args, n_slots, seed):
    gen = torch.Generator().manual_seed(seed)
    table, nbytes = OS.layout(*table_args)
    assert nbytes == lay.nbytes
    raw = torch.randint(0, 256, (n_slots, lay.nbytes), dtype=torch.uint8, generator=gen)
    dev = raw.to(DEV)
    return gen, table, raw, dev


@pytest.mark.parametrize('fmt', [(8, 'k', 64), (4, 'k', 32), (4, 'v', 32), (8, 'v', 32), (8, 'v', 64), (4, 'v', 16), 'bf16', 'fp32'])
def test_write_matches_oracle_whole_blob(fmt):
    HV, HK, D, m = 4, 2, 128, 8
    lay = SlotLayout(quantizer(fmt), HV, HK, D, D, m=m, buffer_bits=8)
    ofmt, sdt = ('bf16', torch.float32) if fmt == 'fp32' else (fmt, torch.bfloat16)
    gen, table, raw, dev = _blob_pair(lay, ('gdn', ofmt, HV, HK, D, D, m, 8, sdt), 9, 1)
    idx = torch.tensor([7, 2, 5])
    S = torch.randn(3, HV, D, D, generator=gen)
    lay.write(lay.views(dev), idx.to(DEV), S.to(DEV))
    OS.write(OS.views(table, raw), idx, S, ofmt, HV, D, D)
    assert torch.equal(dev.cpu(), raw)                    # codes, scales, counters, decays -- and nothing else


def _advance(lay, views, step_fn, schedule):
    """Run decode steps so that the slots end with different buffer fills (schedule: list of slot lists)."""
    for live in schedule:
        step_fn(torch.tensor(live, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize('fmt,bb', [((8, 'k', 128), 8), ((4, 'k', 32), 16), ((4, 'v', 32), 8), ((8, 'v', 32), 16), ((4, 'v', 64), 8),
                                    ('bf16', 8), ('fp32', 16)])
def test_gdn_read_matches_oracle(fmt, bb):
    HV, HK, D, m = 4, 2, 128, 8
    lay = SlotLayout(quantizer(fmt), HV, HK, D, D, m=m, buffer_bits=bb)
    ofmt, sdt = ('bf16', torch.float32) if fmt == 'fp32' else (fmt, torch.bfloat16)
    gen, table, raw, dev = _blob_pair(lay, ('gdn', ofmt, HV, HK, D, D, m, bb, sdt), 6, 2)
    views = lay.views(dev)
    slots = torch.tensor([1, 3, 4, 5])
    lay.write(views, slots.to(DEV), (torch.randn(4, HV, D, D, generator=gen) * 0.5).to(DEV))

    def step(idx):
        B = idx.shape[0]
        q, k, v, g, beta = (x.to(DEV) for x in gdn_token(gen, B, HV, HK, D, D))
        lay.step(views, idx, q, k, v, torch.empty(B, HV, D, device=DEV), D ** -0.5, g=g, beta=beta)

    _advance(lay, views, step, [[1, 3, 4]] * 3 + [[3, 4]] * 2 + [[4]] * 5)         # fills 3, 5, 10 % 8 = 2, 0
    got = lay.read(views, slots.to(DEV)).cpu()
    want = OS.read(OS.views(table, dev.cpu()), slots, ofmt, HV, HK, D, D, m)
    assert (views['NPTR'][slots.to(DEV), 0].cpu() & (m - 1)).tolist() == [3, 5, 2, 0]
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6 * want.abs().max().item())


@pytest.mark.parametrize('fmt', [(4, 'k', 32), (8, 'v', 32), (8, 'v', 16), 'bf16'])
def test_kda_read_matches_oracle(fmt):
    H, DK, DV, m = 4, 128, 128, 8
    lay = KDASlotLayout(quantizer(fmt), H, DK, DV, m=m, buffer_bits=8)
    gen, table, raw, dev = _blob_pair(lay, ('kda', fmt, H, H, DK, DV, m, 8), 5, 3)
    views = lay.views(dev)
    slots = torch.tensor([2, 4, 1])
    lay.write(views, slots.to(DEV), (torch.randn(3, H, DV, DK, generator=gen) * 0.5).to(DEV))
    assert torch.equal(views['GCUR'][slots.to(DEV)].cpu(), torch.zeros(3, H, DK))

    def step(idx):
        B = idx.shape[0]
        q, k, v, g, beta = (x.to(DEV) for x in kda_token(gen, B, H, DK, DV))
        lay.step(views, idx, q, k, v, g, beta, torch.empty(B, H, DV, device=DEV))

    _advance(lay, views, step, [[2, 4]] * 4 + [[4]] * 3)
    got = lay.read(views, slots.to(DEV)).cpu()
    want = OS.read(OS.views(table, dev.cpu()), slots, fmt, H, H, DK, DV, m, per_channel=True)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6 * want.abs().max().item())


@pytest.mark.parametrize('fmt', [(8, 'k', 128), (4, 'v', 32), (4, 'v', 16), 'bf16'])
def test_mamba2_read_matches_oracle(fmt):
    H, G, DK, DV, m = 8, 2, 128, 64, 8
    lay = Mamba2SlotLayout(quantizer(fmt), H, G, DK, DV, m=m, buffer_bits=8)
    gen, table, raw, dev = _blob_pair(lay, ('mamba2', fmt, H, G, DK, DV, m, 8), 5, 4)
    views = lay.views(dev)
    slots = torch.tensor([3, 1])
    lay.write(views, slots.to(DEV), (torch.randn(2, H, DV, DK, generator=gen) * 0.5).to(DEV))
    A, D, dtb = (t.to(DEV) for t in params(gen, H))

    def step(idx):
        B = idx.shape[0]
        x, dt, Bm, C = (t.to(DEV) for t in m2_token(gen, B, H, G, DK, DV))
        lay.step(views, idx, x, dt, Bm, C, torch.empty(B, H, DV, device=DEV), A, D, dtb)

    _advance(lay, views, step, [[3, 1]] * 2 + [[1]] * 4)
    got = lay.read(views, slots.to(DEV)).cpu()
    want = OS.read(OS.views(table, dev.cpu()), slots, fmt, H, G, DK, DV, m)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6 * want.abs().max().item())


def test_padding_rows_in_read_and_write_and_a_host_index():
    """`read` / `write` on a GPU blob: the slot indices may live on the host (the reference indexes with whatever
    tensor it is given); rows with ``idx <= 0`` are padding -- `write` stores nothing for them, `read` returns zeros
    (not uninitialised memory)."""
    HV, HK, D, m = 4, 2, 128, 8
    lay = SlotLayout(quantizer((8, 'k', 64)), HV, HK, D, D, m=m, buffer_bits=8)
    gen = torch.Generator().manual_seed(7)
    blob = torch.randint(0, 256, (6, lay.nbytes), dtype=torch.uint8, generator=gen).to(DEV)
    before = blob.clone()
    views = lay.views(blob)
    idx = torch.tensor([3, 0, 5, -1])                                      # on the host
    S = torch.randn(4, HV, D, D, generator=gen)
    lay.write(views, idx, S)                                               # S on the host as well
    untouched = torch.tensor([0, 1, 2, 4])
    assert torch.equal(blob[untouched.to(DEV)], before[untouched.to(DEV)])
    got = lay.read(views, idx)
    assert got.is_cuda
    twin = lay.views(before.clone())
    lay.write(twin, idx[[0, 2]].to(DEV), S[[0, 2]].to(DEV))
    want = lay.read(twin, idx[[0, 2]].to(DEV))
    assert torch.equal(got[[0, 2]], want)
    assert torch.equal(got[[1, 3]], torch.zeros(2, HV, D, D, device=DEV))
    for _ in range(3):                                                     # fresh allocations: still zeros
        assert torch.equal(lay.read(views, idx)[[1, 3]], torch.zeros(2, HV, D, D, device=DEV))


def test_step_refuses_a_host_operand():
    """`step` takes raw pointers, so an operand that is not on the state's device is refused in Python."""
    HV, HK, D = 4, 2, 128
    lay = SlotLayout(quantizer((8, 'k', 128)), HV, HK, D, D, m=4)
    views = lay.views(lay.alloc(3, DEV))
    q, k, v, g, beta = (x.to(DEV) for x in gdn_token(torch.Generator().manual_seed(1), 2, HV, HK, D, D))
    out = torch.zeros(2, HV, D, device=DEV)
    with pytest.raises(RuntimeError, match='`idx` is on cpu'):
        lay.step(views, torch.tensor([1, 2], dtype=torch.int32), q, k, v, out, 1.0, g=g, beta=beta)
    with pytest.raises(RuntimeError, match='`beta` is on cpu'):
        lay.step(views, torch.tensor([1, 2], dtype=torch.int32, device=DEV), q, k, v, out, 1.0, g=g, beta=beta.cpu())
    assert torch.equal(views['NPTR'], torch.zeros_like(views['NPTR']))


def test_unsupported_layout_raises_instead_of_falling_back(monkeypatch):
    """A GPU blob never takes the torch formulation: `read` / `write` / `pack_vk` either run the HIP kernels or
    raise.  The torch helpers are made to fail here, and every parametrised format above still passes through
    `_hip.pack_into` / `_hip.read_state`."""
    import statequant_amd.kernels.slots as SL
    monkeypatch.setattr(SL, 'pack_vk', lambda *a, **k: (_ for _ in ()).throw(AssertionError('torch path taken')))
    monkeypatch.setattr(SL.SlotLayout, '_stored', lambda *a, **k: (_ for _ in ()).throw(AssertionError('torch path taken')))
    for fmt in [(8, 'k', 128), (4, 'k', 32), (4, 'v', 32), (8, 'v', 16), 'bf16', 'fp32']:
        lay = SlotLayout(quantizer(fmt), 4, 2, 128, 128, m=8)
        views = lay.views(lay.alloc(3, DEV))
        idx = torch.tensor([1, 2], device=DEV)
        lay.write(views, idx, torch.randn(2, 4, 128, 128, device=DEV))
        assert torch.isfinite(lay.read(views, idx)).all()
    lay = SlotLayout(quantizer((8, 'k', 128)), 4, 2, 128, 128, m=32)       # the read kernel stops at m = 16
    views = lay.views(lay.alloc(3, DEV))
    with pytest.raises(RuntimeError, match='libsqhip'):
        lay.read(views, torch.tensor([1], device=DEV))
