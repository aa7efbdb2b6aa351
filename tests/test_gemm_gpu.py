"""GPU parity of the einsum contraction (MFMA kernel and scalar fallback) against
numpy.einsum in fp64 on the same fp16-rounded operands, for all 18 contractions
of the layer under the MI355X layouts and both layouts the reference ships.
fp16 products accumulate in fp32 and are rounded once: tolerance 1e-2 relative."""
import numpy as np
import pytest
import torch

from tests.einsums import EINSUMS, operand_layouts
from tests.helpers import assert_close, from_layout, h16, to_layout

pytestmark = pytest.mark.gpu


def _layout_sets():
    from substation_amd import layouts as L
    return [('mi355x', L.mi355x_layouts()), ('ref-b8', L.reference_layouts('bert-b8-l512-h16-e1024')),
            ('ref-b96', L.reference_layouts('bert-b96-l128-h16-e1024'))]


@pytest.mark.parametrize('B,L,H,E', [(2, 16, 2, 32), (3, 40, 3, 24), (2, 128, 4, 256), (1, 256, 2, 128)])
def test_all_contractions(B, L, H, E):
    from substation_amd.ops import Ops
    o = Ops(B, L, H, E)
    sz = o.sizes
    rng = np.random.default_rng(7)
    kinds = set()
    for lname, lay in _layout_sets():
        t = operand_layouts(lay)
        for name, a, b, c, scaled in EINSUMS:
            la, lb, lc = t[a], t[b], t[c]
            A = h16(rng.normal(size=tuple(sz[d] for d in la)))
            Bm = h16(rng.normal(size=tuple(sz[d] for d in lb)))
            alpha = 1.0 / np.sqrt(sz['P']) if scaled else 1.0
            want = alpha * np.einsum(f'{la},{lb}->{lc}'.lower(), A, Bm)
            C = torch.full(tuple(sz[d] for d in lc), float('nan'), dtype=torch.float16, device='cuda')
            kinds.add(o.handle.classify(la, lb, lc)['kernel'])
            o.einsum(to_layout(A, la, la), la, to_layout(Bm, lb, lb), lb, C, lc, alpha=alpha)
            torch.cuda.synchronize()
            assert_close(from_layout(C, lc, lc), want, name=f'{lname}:{name} {la},{lb}->{lc}')
    if E % 8 == 0 and L % 8 == 0:
        assert 1 in kinds, 'the MFMA kernel was never selected'


def test_k_remainder_and_tile_edges():
    """K not a multiple of the 64-wide LDS tile, M/N not multiples of 128."""
    from substation_amd.ops import Ops
    o = Ops(3, 72, 5, 200)          # P=40, U=800
    sz = o.sizes
    rng = np.random.default_rng(8)
    for la, lb, lc in (('BJI', 'UI', 'BJU'), ('BJU', 'IU', 'BJI'), ('BJI', 'BJU', 'UI'),
                       ('BKHP', 'BJHP', 'BHJK'), ('BHJK', 'BKHP', 'BJHP'), ('BJHP', 'BHJK', 'BKHP')):
        A = h16(rng.normal(size=tuple(sz[d] for d in la)))
        Bm = h16(rng.normal(size=tuple(sz[d] for d in lb)))
        want = np.einsum(f'{la},{lb}->{lc}'.lower(), A, Bm)
        C = torch.full(tuple(sz[d] for d in lc), float('nan'), dtype=torch.float16, device='cuda')
        assert o.handle.classify(la, lb, lc)['kernel'] == 1
        o.einsum(to_layout(A, la, la), la, to_layout(Bm, lb, lb), lb, C, lc)
        torch.cuda.synchronize()
        assert_close(from_layout(C, lc, lc), want, name=f'{la},{lb}->{lc}')


@pytest.mark.parametrize('E,H', [(192, 3), (64, 1), (128, 2)])
def test_wide_tiles_every_operand_orientation(E, H):
    """4096 x 4096 outputs take the 256 x 256 tiles of the asynchronous kernel with
    eight waves: each operand k-contiguous or not, with an odd number of 64-deep
    k-tiles (three, one) and an even one."""
    from substation_amd.ops import Ops
    o = Ops(8, 512, H, E, intermediate_size=4096)
    sz = o.sizes
    rng = np.random.default_rng(E)
    for la in ('BJI', 'IBJ'):
        for lb in ('UI', 'IU'):
            lc = 'BJU'
            A = h16(rng.normal(size=tuple(sz[d] for d in la)))
            Bm = h16(rng.normal(size=tuple(sz[d] for d in lb)))
            want = np.einsum(f'{la},{lb}->{lc}'.lower(), A, Bm)
            C = torch.full(tuple(sz[d] for d in lc), float('nan'), dtype=torch.float16, device='cuda')
            assert o.handle.classify(la, lb, lc)['kernel'] == 1
            o.einsum(to_layout(A, la, la), la, to_layout(Bm, lb, lb), lb, C, lc)
            torch.cuda.synchronize()
            assert_close(from_layout(C, lc, lc), want, name=f'{la},{lb}->{lc} K={E}')
