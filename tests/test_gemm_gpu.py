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


@pytest.mark.parametrize('B,L,H,E,expect_pair', [(8, 512, 16, 1024, True), (2, 128, 4, 256, False)])
def test_two_contractions_in_one_call(B, L, H, E, expect_pair):
    """sub_op_einsum_pair: a data gradient (with and without a residual added in its
    epilogue) and the weight gradient next to it, as one launch at the bench workload's
    sizes, and at small sizes (paired or not, as the launcher decides); either way against
    numpy.einsum and equal to what the two single calls give (to rounding where a
    small output's contraction is split differently)."""
    from substation_amd.ops import Ops
    o = Ops(B, L, H, E)
    sz = o.sizes
    rng = np.random.default_rng(11)
    mk = lambda lay, s=1.0: h16(s * rng.normal(size=tuple(sz[d] for d in lay)))
    nan = lambda lay: torch.full(tuple(sz[d] for d in lay), float('nan'), dtype=torch.float16, device='cuda')
    cases = [
        # dXlin1 + dWlin1
        (('BJU', 'UI', 'BJI', None), ('BJU', 'BJI', 'UI')),
        # dXQKV + residual, dWQKV
        (('QHPI', 'QBJHP', 'BJI', 'BJI'), ('QBJHP', 'BJI', 'QHPI')),
        # dXout, dWout
        (('IHP', 'BJI', 'BJHP', None), ('BJI', 'BJHP', 'IHP')),
    ]
    for (la1, lb1, lc1, lt1), (la2, lb2, lc2) in cases:
        # the shared operand is the same tensor in both products, as in a backward pass
        shared = {}
        def operand(lay, s=1.0):
            if lay not in shared:
                shared[lay] = mk(lay, s)
            return shared[lay]
        A1, B1 = operand(la1, 0.5), operand(lb1, 0.5)
        A2, B2 = operand(la2, 0.5), operand(lb2, 0.5)
        T1 = mk(lt1) if lt1 else None
        want1 = np.einsum(f'{la1},{lb1}->{lc1}'.lower(), A1, B1) + (T1 if lt1 else 0)
        want2 = np.einsum(f'{la2},{lb2}->{lc2}'.lower(), A2, B2)
        dev = {k: to_layout(v, k, k) for k, v in shared.items()}
        t1 = to_layout(T1, lt1, lt1) if lt1 else None
        C1, C2 = nan(lc1), nan(lc2)
        first = (dev[la1], la1, dev[lb1], lb1, C1, lc1) + ((t1, lt1) if lt1 else ())
        paired = o.einsum_pair(first, (dev[la2], la2, dev[lb2], lb2, C2, lc2))
        torch.cuda.synchronize()
        S1, S2 = nan(lc1), nan(lc2)
        o.einsum(dev[la1], la1, dev[lb1], lb1, S1, lc1, addend=t1, l_addend=lt1)
        o.einsum(dev[la2], la2, dev[lb2], lb2, S2, lc2)
        torch.cuda.synchronize()
        name = f'{la1},{lb1}->{lc1} + {la2},{lb2}->{lc2}'
        assert_close(from_layout(C1, lc1, lc1), want1, name=name + ' (first)')
        assert_close(from_layout(C2, lc2, lc2), want2, name=name + ' (second)')
        assert_close(C1.float().cpu().numpy(), S1.float().cpu().numpy(), tol=2e-3, name=name + ' first vs single')
        assert_close(C2.float().cpu().numpy(), S2.float().cpu().numpy(), tol=2e-3, name=name + ' second vs single')
    if expect_pair:
        # the pair the layer itself launches must have gone out as one launch here too
        la1, lb1, lc1 = 'BJU', 'UI', 'BJI'
        la2, lb2, lc2 = 'BJU', 'BJI', 'UI'
        d = {k: to_layout(mk(k, 0.5), k, k) for k in ('BJU', 'UI', 'BJI')}
        assert o.einsum_pair((d['BJU'], 'BJU', d['UI'], 'UI', nan('BJI'), 'BJI'),
                             (d['BJU'], 'BJU', d['BJI'], 'BJI', nan('UI'), 'UI'))
