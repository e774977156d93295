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


# ---------------------------------------------------------------------------------------------------------------
# The patches themselves, on stand-in engine modules (no engine installed): the state calculators answer packed only
# to the callers whose layers have a packed forward, the GDN base class refuses other subclasses, the patched
# constructors attach the layout and refuse unsupported cache settings, and everything can be undone.
# ---------------------------------------------------------------------------------------------------------------
import types  # noqa: E402

from statequant_amd.integrations import vllm_olmo  # noqa: E402


def _fake_mamba_utils():
    class MambaStateShapeCalculator:
        @classmethod
        def gated_delta_net_state_shape(cls, tp, nk, nv, dk, dv, conv_kernel_size, num_spec=0):
            return ((2 * nk * dk + nv * dv) // tp, conv_kernel_size - 1), (nv // tp, dv, dk)

        @classmethod
        def kda_state_shape(cls, tp, num_heads, head_dim, num_k_heads=None, head_k_dim=None, conv_kernel_size=4,
                            num_spec=0):
            return (3 * num_heads * head_dim // tp, conv_kernel_size - 1), (num_heads // tp, head_dim, head_dim)

        @classmethod
        def mamba2_state_shape(cls, tp_world_size, intermediate_size, n_groups, num_heads, head_dim, state_size,
                               conv_kernel, num_spec=0):
            return ((intermediate_size + 2 * n_groups * state_size) // tp_world_size, conv_kernel - 1), \
                (num_heads // tp_world_size, head_dim, state_size)

    class MambaStateDtypeCalculator:
        @classmethod
        def gated_delta_net_state_dtype(cls, model_dtype, mamba_cache_dtype, mamba_ssm_cache_dtype='auto'):
            return model_dtype, torch.bfloat16

        @classmethod
        def kda_state_dtype(cls, model_dtype, mamba_cache_dtype, mamba_ssm_cache_dtype='auto'):
            return model_dtype, torch.float32

        @classmethod
        def mamba2_state_dtype(cls, model_dtype, mamba_cache_dtype, mamba_ssm_cache_dtype):
            return model_dtype, torch.float32

    return types.SimpleNamespace(MambaStateShapeCalculator=MambaStateShapeCalculator,
                                 MambaStateDtypeCalculator=MambaStateDtypeCalculator)


def _call_from(module_name, expr, **names):
    """Evaluate ``expr`` in a function whose module is ``module_name`` (what the calculators look at: their caller)."""
    g = dict(names, __name__=module_name, torch=torch)
    exec(f'def hook():\n    return {expr}\n', g)
    return g['hook']()


def _vllm_config(spec=None, prefix_caching=False, mode='none', eager=True):
    return types.SimpleNamespace(speculative_config=spec, model_config=types.SimpleNamespace(enforce_eager=eager),
                                 cache_config=types.SimpleNamespace(enable_prefix_caching=prefix_caching,
                                                                    mamba_cache_mode=mode, mamba_ssm_cache_dtype='auto'))


def test_gdn_calculators_answer_packed_to_supported_callers_only():
    P.configure({'STATEQUANT_VLLM': 'pace4'})
    mu = _fake_mamba_utils()
    P._patch_calculators(mu)
    try:
        shape = 'mu.MambaStateShapeCalculator.gated_delta_net_state_shape(1, 16, 32, 128, 128, 4)'
        dtype = "mu.MambaStateDtypeCalculator.gated_delta_net_state_dtype(torch.bfloat16, 'auto')"
        want = P.layout(32, 16, 128, 128).nbytes
        for mod in P.PACKED_MODEL_MODULES + (P.PACKED_MODEL_MODULES[0] + '.sub',):
            assert _call_from(mod, shape, mu=mu) == ((2 * 16 * 128 + 32 * 128, 3), (want,))
            assert _call_from(mod, dtype, mu=mu) == (torch.bfloat16, torch.uint8)
        # tensor parallel: each rank packs its own heads
        tp2 = 'mu.MambaStateShapeCalculator.gated_delta_net_state_shape(2, 16, 32, 128, 128, 4)'
        assert _call_from(P.PACKED_MODEL_MODULES[1], tp2, mu=mu)[1] == (P.layout(16, 8, 128, 128).nbytes,)
        for mod in ('vllm.model_executor.models.minicpmv', 'vllm.model_executor.models.qwen3_next_mtp'):
            with pytest.raises(NotImplementedError, match='stores packed GDN states only for'):
                _call_from(mod, shape, mu=mu)
            with pytest.raises(NotImplementedError):
                _call_from(mod, dtype, mu=mu)
        # a layer asking through its own method is recognised by its class, whatever module the call comes from
        Layer = type('QwenGatedDeltaNetAttention', (), {'__module__': P.PACKED_LAYER[0]})
        Sub = type('Derived', (Layer,), {'__module__': 'somewhere.else'})
        Other = type('MiniGDN', (), {'__module__': 'vllm.model_executor.layers.mamba.gdn.other'})

        def get_state_shape(self):
            return mu.MambaStateShapeCalculator.gated_delta_net_state_shape(1, 16, 32, 128, 128, 4)
        assert get_state_shape(Sub())[1] == (want,)
        with pytest.raises(NotImplementedError, match='MiniGDN'):
            get_state_shape(Other())
        with pytest.raises(AssertionError, match='speculative'):
            _call_from(P.PACKED_MODEL_MODULES[0],
                       'mu.MambaStateShapeCalculator.gated_delta_net_state_shape(1, 16, 32, 128, 128, 4, 2)', mu=mu)
    finally:
        P.unpatch()
    assert mu.MambaStateShapeCalculator.gated_delta_net_state_shape(1, 16, 32, 128, 128, 4)[1] == (32, 128, 128)


def _fake_gdn_modules():
    class GatedDeltaNetAttention:
        def __init__(self, *a, **k):
            self.base_built = True

    def make(name):
        def __init__(self, config, vllm_config, prefix='model.layers.1.linear_attn'):
            GatedDeltaNetAttention.__init__(self)
            self.prefix, self.tp_size = prefix, 2
            self.num_v_heads, self.num_k_heads, self.head_k_dim, self.head_v_dim = 32, 16, 128, 128
        return type(name, (GatedDeltaNetAttention,), {
            '__init__': __init__, '_forward_core': lambda self, *a: 'stock',
            '_warmup_prefill_kernels': lambda self, qkv, v_dim: self.get_state_dtype(),
            'get_state_dtype': lambda self: (torch.bfloat16, torch.uint8)})
    Q = types.SimpleNamespace(QwenGatedDeltaNetAttention=make('QwenGatedDeltaNetAttention'), logger=None)
    O = types.SimpleNamespace(OlmoHybridGatedDeltaNetAttention=make('OlmoHybridGatedDeltaNetAttention'))
    Other = type('OtherGDN', (GatedDeltaNetAttention,), {'__init__': lambda self: GatedDeltaNetAttention.__init__(self)})
    return Q, O, types.SimpleNamespace(GatedDeltaNetAttention=GatedDeltaNetAttention), Other


def test_gdn_layer_patch_attaches_layout_and_refuses_the_rest():
    P.configure({'STATEQUANT_VLLM': 'int8k'})
    Q, O, base, Other = _fake_gdn_modules()
    cfg = types.SimpleNamespace(layer_types=['linear_attention'] * 4)
    P._patch_layer(Q, O, base)
    vllm_olmo.patch(P.layout, O)
    try:
        P._patch_layer(Q, O, base)                            # idempotent
        layer = Q.QwenGatedDeltaNetAttention(cfg, _vllm_config())
        assert layer.base_built and layer._sq_layout is P.layout(16, 8, 128, 128) and layer._sq_views is None
        assert layer._sq_external is None and layer._sq_lk == {}
        assert Q.QwenGatedDeltaNetAttention._forward_core is P._forward_core
        # the prefill warm-up sees an fp32 state dtype, and the override is gone afterwards
        assert layer._warmup_prefill_kernels(None, 0) == (torch.bfloat16, torch.float32)
        assert layer.get_state_dtype() == (torch.bfloat16, torch.uint8)
        olmo = O.OlmoHybridGatedDeltaNetAttention(cfg, _vllm_config())
        assert olmo._sq_layout is layer._sq_layout and O.OlmoHybridGatedDeltaNetAttention._forward_core is vllm_olmo._forward_core
        with pytest.raises(NotImplementedError, match='OtherGDN'):
            Other()
        for bad, msg in ((_vllm_config(spec=object()), 'speculative'), (_vllm_config(prefix_caching=True), 'prefix caching')):
            with pytest.raises(AssertionError, match=msg):
                Q.QwenGatedDeltaNetAttention(cfg, bad)
            with pytest.raises(AssertionError, match=msg):
                O.OlmoHybridGatedDeltaNetAttention(cfg, bad)
        with pytest.raises(AssertionError):
            Q.QwenGatedDeltaNetAttention(cfg, _vllm_config(mode='align'))
    finally:
        P.unpatch()
        vllm_olmo.unpatch()
    assert Q.QwenGatedDeltaNetAttention(cfg, _vllm_config())._forward_core() == 'stock'
    assert not hasattr(Q.QwenGatedDeltaNetAttention(cfg, _vllm_config()), '_sq_layout')
    Other()


def test_external_quantizer_settings(tmp_path):
    src = tmp_path / 'q.py'
    src.write_text('def halve(S, layer):\n    return S * 0.5 + layer\n\nnot_callable = 3\n')
    P.configure({'STATEQUANT_VLLM': f'external:{src}:halve', 'STATEQUANT_VLLM_EXTERNAL_DTYPE': 'bf16'})
    assert P.layout(4, 2, 64, 64).state_dtype == torch.bfloat16
    S = torch.arange(2 * 3 * 4 * 5, dtype=torch.float32).view(2, 3, 4, 5)           # value-major [P, HV, d_v, d_k]
    got = P.apply_external(S, 2)
    assert got.shape == S.shape and torch.equal(got, S * 0.5 + 2)
    cfg = types.SimpleNamespace(layer_types=['linear_attention', 'full_attention', 'linear_attention'])
    assert P.gdn_ordinal(cfg, 'model.layers.2.linear_attn') == 1 and P.gdn_ordinal(cfg, 'model.layers.0.x') == 0
    with pytest.raises(AssertionError):
        P.gdn_ordinal(cfg, 'model.layers.1.self_attn')
    Q, O, base, _ = _fake_gdn_modules()
    P._patch_layer(Q, O, base)
    try:
        with pytest.raises(AssertionError, match='no tensor parallelism'):           # the fake layers have tp_size 2
            Q.QwenGatedDeltaNetAttention(cfg, _vllm_config(), prefix='model.layers.2.linear_attn')
    finally:
        P.unpatch()
    P.configure({'STATEQUANT_VLLM': f'external:{src}:not_callable'})
    with pytest.raises(AssertionError, match='not callable'):
        P.external_fn()
    P.configure({'STATEQUANT_VLLM': 'external:json:dumps'})                         # an importable module
    import json
    assert P.external_fn() is json.dumps
    P.configure({'STATEQUANT_VLLM': 'off'})
    assert P.external_fn() is None


def test_kda_and_mamba2_patches_are_scoped_to_their_models():
    cfg = P.configure({'STATEQUANT_VLLM': 'pace4'})
    mu = _fake_mamba_utils()
    vllm_kda._patch_calculators(cfg, mu)
    vllm_mamba2._patch_calculators(cfg, mu)
    try:
        kda = 'mu.MambaStateShapeCalculator.kda_state_shape(1, 16, 128)'
        assert _call_from('vllm.model_executor.models.bailing_moe_v3', kda, mu=mu)[1] == (246336,)
        assert _call_from('vllm.model_executor.models.kimi_linear', kda, mu=mu)[1] == (16, 128, 128)  # stock answer
        kd = "mu.MambaStateDtypeCalculator.kda_state_dtype(torch.bfloat16, 'auto')"
        assert _call_from('vllm.model_executor.models.bailing_moe_v3', kd, mu=mu) == (torch.bfloat16, torch.uint8)
        assert _call_from('elsewhere', kd, mu=mu) == (torch.bfloat16, torch.float32)
        with pytest.raises(AssertionError, match='tensor parallel'):
            _call_from('vllm.model_executor.models.bailing_moe_v3',
                       'mu.MambaStateShapeCalculator.kda_state_shape(2, 16, 128)', mu=mu)
        m2 = ('mu.MambaStateShapeCalculator.mamba2_state_shape(tp_world_size=1, intermediate_size=7680, n_groups=8, '
              'num_heads=96, head_dim=80, state_size=128, conv_kernel=4)')
        for mod in ('vllm.model_executor.layers.mamba.mamba_mixer2', 'vllm.model_executor.models.nemotron_h',
                    'vllm.model_executor.models.falcon_h1'):
            assert _call_from(mod, m2, mu=mu)[1] == (597376,)
        assert _call_from('vllm.model_executor.models.plamo2', m2, mu=mu)[1] == (96, 80, 128)
        md = "mu.MambaStateDtypeCalculator.mamba2_state_dtype(torch.bfloat16, 'auto', 'auto')"
        assert _call_from('vllm.model_executor.models.zamba2', md, mu=mu) == (torch.bfloat16, torch.uint8)
        assert _call_from('vllm.model_executor.models.plamo2', md, mu=mu) == (torch.bfloat16, torch.float32)
    finally:
        vllm_kda.unpatch()
        vllm_mamba2.unpatch()
    assert mu.MambaStateShapeCalculator.kda_state_shape(1, 16, 128)[1] == (16, 128, 128)


def test_kda_and_mamba2_layer_patches():
    cfg = P.configure({'STATEQUANT_VLLM': 'int8k'})
    box = {'vc': _vllm_config()}

    class Kimi:
        def __init__(self, config, tp=1, spec=0):
            self.tp_size, self.num_speculative_tokens, self.local_num_heads, self.head_dim = tp, spec, 16, 128

        def _forward(self, *a):
            return 'stock'
    Mk = types.SimpleNamespace(BailingMoeV3KimiDeltaAttention=Kimi, get_current_vllm_config=lambda: box['vc'])

    class Mixer:
        def __init__(self, tp=1, replay=False):
            self.tp_size, self.num_spec, self.use_replayssm = tp, 0, replay
            self.num_heads, self.n_groups, self.ssm_state_size, self.head_dim = 96, 8, 128, 80

        def _warmup_ssd_kernels(self, ps):
            return self.get_state_dtype()

        def get_state_dtype(self):
            return (torch.bfloat16, torch.uint8)

        def conv_ssm_forward(self, *a):
            return 'stock'
    Mm = types.SimpleNamespace(MambaMixer2=Mixer, get_current_vllm_config=lambda: box['vc'], logger=None)
    vllm_kda._patch_layer(cfg, Mk)
    vllm_mamba2._patch_layer(cfg, Mm)
    try:
        k = Kimi(None)
        assert k._sq_layout is vllm_kda.layout(cfg, 16, 128) and Kimi._forward is vllm_kda._forward
        with pytest.raises(AssertionError, match='tensor parallel'):
            Kimi(None, tp=2)
        with pytest.raises(AssertionError, match='MTP'):
            Kimi(None, spec=1)
        mx = Mixer()
        assert mx._sq_layout is vllm_mamba2.layout(cfg, 96, 8, 128, 80) and Mixer.conv_ssm_forward is vllm_mamba2.conv_ssm_forward
        assert mx._warmup_ssd_kernels(None) == (torch.bfloat16, torch.float32) and mx.get_state_dtype()[1] == torch.uint8
        with pytest.raises(AssertionError, match='ReplaySSM'):
            Mixer(replay=True)
        with pytest.raises(AssertionError, match='tensor parallel'):
            Mixer(tp=2)
        box['vc'] = _vllm_config(prefix_caching=True)
        with pytest.raises(AssertionError, match='prefix caching'):
            Mixer()
        with pytest.raises(AssertionError, match='prefix caching'):
            Kimi(None)
    finally:
        vllm_kda.unpatch()
        vllm_mamba2.unpatch()
    box['vc'] = _vllm_config()
    assert Kimi(None)._forward() == 'stock' and Mixer().conv_ssm_forward() == 'stock'


def test_register_is_a_no_op_when_off(monkeypatch):
    monkeypatch.delenv('STATEQUANT_VLLM', raising=False)
    P.register()                                               # off: nothing imported, nothing patched
    assert 'registered' not in P._state
    monkeypatch.setenv('STATEQUANT_VLLM', 'pace4')
    with pytest.raises(ImportError):                           # on, and no engine installed here
        P.register()
    P.unpatch()
    P.configure({'STATEQUANT_VLLM': 'off'})
