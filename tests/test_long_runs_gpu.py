"""Long decode runs: a thousand and more tokens per configuration, kernel against oracle with the reference's re-sync
after every fold, so that rare events (a code or a buffered value on a rounding tie, a scale on an fp16 boundary) are
counted over tens of millions of codes.  Bounds: the task's (outputs, codes >= 99.9 % identical, none further than one
step), with the measured rates two to three orders of magnitude below them."""
import pytest

from tests import test_gdn_gpu as G
from tests import test_kda_gpu as K
from tests import test_mamba2_gpu as M

pytestmark = pytest.mark.gpu


def verdict(t, tag):
    print('\n' + t.report(tag))
    assert t.worst_o < 1e-4, t.worst_o
    assert t.code_far == 0
    assert t.code_mism <= 1e-4 * t.code_n, (t.code_mism, t.code_n)
    assert t.buf_flips <= 1e-3 * t.buf_entries, (t.buf_flips, t.buf_entries)
    assert t.buf_scale_events * 64 <= 1e-2 * t.buf_entries, (t.buf_scale_events, t.buf_entries)   # <= 1 % of the vectors


@pytest.mark.parametrize('fmt,m,bb', [((8, 'k', 128), 8, 8), ((4, 'k', 64), 8, 8), ((4, 'k', 32), 16, 16), ((8, 'v', 32), 8, 8),
                                      ((4, 'v', 16), 4, 8), ('bf16', 8, 8)])
def test_gdn_two_thousand_tokens(fmt, m, bb):
    verdict(G.run_decode(fmt, m, bb, T=2000, seed=7), f'gdn {fmt} m={m} buf{bb}, 2000 tokens')


@pytest.mark.parametrize('fmt,m,bb', [((4, 'k', 32), 8, 8), ((8, 'k', 64), 16, 16), ((4, 'v', 32), 8, 8)])
def test_kda_thousand_tokens(fmt, m, bb):
    verdict(K.run_decode(fmt, m, bb, T=1000, seed=7), f'kda {fmt} m={m} buf{bb}, 1000 tokens')


@pytest.mark.parametrize('fmt,m,bb', [((8, 'k', 128), 8, 8), ((4, 'k', 32), 8, 16), ((8, 'v', 16), 8, 8)])
def test_mamba2_thousand_tokens_head_dim_80(fmt, m, bb):
    verdict(M.run_decode(fmt, m, bb, T=1000, seed=7, DK=128, DV=80, H=6, G=2), f'mamba2 128x80 {fmt} m={m} buf{bb}, 1000 tokens')
