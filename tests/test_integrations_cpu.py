"""The engine-facing glue that needs no engine: environment strings -> storage configuration -> slot layouts -> the
byte counts the reference documents for its end-to-end runs (docs/vllm.md:117, :145, :190 there), the layer-kind
selection (tests/test_vllm_mamba2_plugin.py:68-80 there) and the asserted restrictions (TP = 1, no speculative
decoding for Mamba2 / KDA)."""
import pytest
import torch

import statequant_amd as sq
from statequant_amd.integrations import vllm_kda, vllm_mamba2, vllm_plugin as P
from statequant_amd.kernels import KDASlotLayout, Mamba2SlotLayout, SlotLayout
from statequant_amd.kernels.gga import GGAPacked


@pytest.mark.parametrize('value', ['', '0', 'off', 'none', 'stock', ' OFF '])
def test_off_is_off(value):
    assert P.config({'STATEQUANT_VLLM': value}) is None
    assert P.configure({'STATEQUANT_VLLM': value}) is None and P.active_kinds() == ()
    assert P.config({}) is None


@pytest.mark.parametrize('name,triple', [('pace4', (4, 'k', 64)), ('int4k', (4, 'k', 64)), ('int4v', (4, 'v', 32)),
                                         ('int8k', (8, 'k', 32)), ('int8v', (8, 'v', 32)), ('INT8K', (8, 'k', 32)),
                                         ('int4kg32', (4, 'k', 32)), ('int8vg16', (8, 'v', 16)), ('int4kg128', (4, 'k', 128))])
def test_presets_and_spelled_formats(name, triple):
    fmt, m, bb, fused = P.config({'STATEQUANT_VLLM': name})
    assert (fmt.bits, fmt.axis, fmt.group) == triple and (m, bb, fused) == (8, 8, None)


def test_settings_and_errors():
    env = {'STATEQUANT_VLLM': 'bf16', 'STATEQUANT_VLLM_M': '16', 'STATEQUANT_VLLM_BUFFER_BITS': '16',
           'STATEQUANT_VLLM_FUSED': '1'}
    assert P.config(env) == ('bf16', 16, 16, True)
    assert P.config(dict(env, STATEQUANT_VLLM='fp32', STATEQUANT_VLLM_FUSED='0')) == ('fp32', 16, 16, False)
    for bad in ('int5kg32', 'int4xg32', 'pace', 'int4k32'):
        with pytest.raises(AssertionError, match='use pace4'):
            P.config({'STATEQUANT_VLLM': bad})
    with pytest.raises(AssertionError, match='0, 1 or auto'):
        P.config({'STATEQUANT_VLLM': 'pace4', 'STATEQUANT_VLLM_FUSED': 'yes'})
    with pytest.raises(AssertionError, match='no plan file'):
        P.config({'STATEQUANT_VLLM': 'gga:/nonexistent/plan.pt:pw'})
    # external:<src>:<fn>: an unpacked slot state in the named dtype, GDN layers only
    assert P.config({'STATEQUANT_VLLM': 'external:pkg.mod:fn'})[0] == 'fp32'
    assert P.config({'STATEQUANT_VLLM': 'external:/x/q.py:fn', 'STATEQUANT_VLLM_EXTERNAL_DTYPE': 'BF16'})[0] == 'bf16'
    with pytest.raises(AssertionError, match='external:<file.py or module>:<function>'):
        P.config({'STATEQUANT_VLLM': 'external:fn'})
    with pytest.raises(AssertionError, match='fp32 or bf16'):
        P.config({'STATEQUANT_VLLM': 'external:m:fn', 'STATEQUANT_VLLM_EXTERNAL_DTYPE': 'fp16'})
    P.configure({'STATEQUANT_VLLM': 'external:m:fn'})
    assert P.active_kinds() == ('gdn',)
    with pytest.raises(AssertionError, match='GDN layers only'):
        P.configure({'STATEQUANT_VLLM': 'external:m:fn', 'STATEQUANT_VLLM_LAYERS': 'mamba2'})
    P.configure({'STATEQUANT_VLLM': 'off'})


def test_layer_kinds():
    assert P.layer_kinds({}) == ('gdn', 'mamba2', 'kda')
    assert P.layer_kinds({'STATEQUANT_VLLM_LAYERS': 'mamba2'}) == ('mamba2',)
    assert P.layer_kinds({'STATEQUANT_VLLM_LAYERS': 'gdn, mamba2'}) == ('gdn', 'mamba2')
    assert P.layer_kinds({'STATEQUANT_VLLM_LAYERS': 'KDA,mamba2'}) == ('kda', 'mamba2')
    with pytest.raises(AssertionError, match='lightning'):
        P.layer_kinds({'STATEQUANT_VLLM_LAYERS': 'lightning'})
    P.configure({'STATEQUANT_VLLM': 'fp32'})
    assert P.active_kinds() == ('gdn',)                       # fp32 (and gga) states: GDN layers only
    with pytest.raises(AssertionError, match='GDN layers only'):
        P.configure({'STATEQUANT_VLLM': 'fp32', 'STATEQUANT_VLLM_LAYERS': 'gdn,kda'})


# the reference's end-to-end tables: bytes per slot and layer of the packed recurrent state
QWEN = dict(num_k_heads=16, num_v_heads=32, head_k_dim=128, head_v_dim=128)
OLMO = dict(num_k_heads=30, num_v_heads=30, head_k_dim=96, head_v_dim=192)
NANO = dict(n_groups=8, num_heads=96, head_dim=80, state_size=128)


@pytest.mark.parametrize('env,want', [('pace4', 370816), ('int8k', 658816), ('int4v', 382336), ('bf16', 1177216)])
def test_olmo_hybrid_slot_bytes(env, want):
    P.configure({'STATEQUANT_VLLM': env})
    assert P.gated_delta_net_state_shape(1, **OLMO) == (want,)
    assert P.state_dtype() == torch.uint8


@pytest.mark.parametrize('env,want', [('pace4', 597376), ('int8k', 1119616), ('int4v', 689536), ('bf16', 2041216)])
def test_nemotron_nano_slot_bytes(env, want):
    cfg = P.configure({'STATEQUANT_VLLM': env})
    assert vllm_mamba2.mamba2_state_shape(cfg, 1, **NANO) == (want,)
    lay = vllm_mamba2.layout(cfg, 96, 8, 128, 80)
    assert isinstance(lay, Mamba2SlotLayout)
    if env == 'int4v':                                        # value-axis group 32 does not divide head_dim 80
        assert (lay.fmt.axis, lay.fmt.group) == ('v', 16)


@pytest.mark.parametrize('env,want', [('pace4', 246336), ('int8k', 385600), ('int4v', 254528), ('bf16', 631360)])
def test_ling_kda_slot_bytes(env, want):
    cfg = P.configure({'STATEQUANT_VLLM': env})
    assert vllm_kda.kda_state_shape(cfg, 1, 16, 128) == (want,)
    assert vllm_kda.kda_state_shape(cfg, 1, 16, 128, num_k_heads=16, head_k_dim=128) == (want,)
    assert isinstance(vllm_kda.layout(cfg, 16, 128), KDASlotLayout) and vllm_kda.state_dtype() == torch.uint8


def test_layout_cache_and_tensor_parallel_split():
    P.configure({'STATEQUANT_VLLM': 'int8k', 'STATEQUANT_VLLM_M': '4'})
    a = P.layout(32, 16, 128, 128)
    assert P.layout(32, 16, 128, 128) is a and isinstance(a, SlotLayout) and a.m == 4
    assert P.layout(16, 8, 128, 128) is not a
    # GDN heads split over ranks: each rank's blob holds its own heads
    assert P.gated_delta_net_state_shape(2, **QWEN) == (P.layout(16, 8, 128, 128).nbytes,)
    assert P.gated_delta_net_state_shape(1, **QWEN) == (a.nbytes,)
    with pytest.raises(AssertionError, match='speculative'):
        P.gated_delta_net_state_shape(1, **QWEN, num_spec=2)
    P.configure({'STATEQUANT_VLLM': 'int8k'})                  # a new configuration drops the cached layouts
    assert P.layout(32, 16, 128, 128) is not a and P.layout(32, 16, 128, 128).m == 8


def test_mamba2_and_kda_restrictions():
    cfg = P.configure({'STATEQUANT_VLLM': 'pace4'})
    with pytest.raises(AssertionError, match='tensor parallel'):
        vllm_mamba2.mamba2_state_shape(cfg, 2, **NANO)
    with pytest.raises(AssertionError, match='speculative'):
        vllm_mamba2.mamba2_state_shape(cfg, 1, **NANO, num_spec=1)
    with pytest.raises(AssertionError, match='tensor parallel'):
        vllm_kda.kda_state_shape(cfg, 2, 16, 128)
    with pytest.raises(AssertionError, match='MTP'):
        vllm_kda.kda_state_shape(cfg, 1, 16, 128, num_spec=1)
    with pytest.raises(AssertionError):
        vllm_kda.kda_state_shape(cfg, 1, 16, 128, num_k_heads=8)


@pytest.mark.parametrize('fmt,dk,dv,group', [((4, 'v', 32), 128, 80, 16), ((8, 'v', 64), 128, 80, 16), ((4, 'v', 32), 128, 64, 32),
                                             ((4, 'k', 64), 96, 80, 32), ((8, 'k', 32), 128, 80, 32), ((4, 'v', 32), 128, 6, 2)])
def test_fmt_for_halves_the_group_until_it_divides(fmt, dk, dv, group):
    q = sq.Quantizer(*fmt)
    got = vllm_mamba2._fmt_for(q, dk, dv)
    assert (got.bits, got.axis, got.group) == (fmt[0], fmt[1], group)
    if group == fmt[2]:
        assert got is q
    assert vllm_mamba2._fmt_for('bf16', dk, dv) == 'bf16'


def test_gga_plan_file(tmp_path):
    """``gga:<plan.pt>[:pw]``: the plan file is read with the safe loader, one GGAPacked per head geometry."""
    HV, D = 32, 128
    widths = torch.tensor(([2] * 12 + [4] * 11 + [6] * 6 + [8] * 2 + [16])[:HV])
    path = tmp_path / 'plan.pt'
    torch.save({'class': 'GGA', 'bits': 4, 'group': 32, 'pivots': 1, 'candidates': None,
                'plan': {0: (widths, torch.ones(HV, D))}}, path)
    cfg = P.configure({'STATEQUANT_VLLM': f'gga:{path}:pw', 'STATEQUANT_VLLM_PW_M': '4'})
    assert cfg[0] == 'gga' and P.gga_settings() == (str(path), True, 4) and P.active_kinds() == ('gdn',)
    lay = P.layout(HV, 16, D, D)
    assert isinstance(lay, GGAPacked) and lay.pw and lay.m == 4 and P.layout(HV, 16, D, D) is lay
    assert P.gated_delta_net_state_shape(1, **QWEN) == (lay.nbytes,)
    cfg = P.configure({'STATEQUANT_VLLM': f'gga:{path}'})
    assert P.gga_settings()[1] is False and not P.layout(HV, 16, D, D).pw
