"""The oracle against the committed fixtures (tests/golden/*.npz)."""
import os

import numpy as np
import pytest

from oracle import encoder_ref as ref
from oracle import philox_ref as ph

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')


def load_encoder_fixture(act):
    z = np.load(os.path.join(GOLD, f'encoder_b2_l8_h2_e16_{act}.npz'))
    params = {k[6:]: z[k] for k in z.files if k.startswith('param_')}
    masks = {k[5:]: z[k].astype(np.float64) for k in z.files if k.startswith('mask_')}
    want = {k[4:]: z[k] for k in z.files if k.startswith('out_')}
    return params, z['in_X'], z['in_DY'], masks, want


@pytest.mark.parametrize('act', ['relu', 'gelu'])
def test_oracle_matches_encoder_fixture(act):
    params, X, DY, masks, want = load_encoder_fixture(act)
    got = ref.run_named(params, X, DY, masks, act)
    assert len(want) >= 23 + 14 + 12 + 2 - 4     # masks are inputs, not outputs
    for name, w in want.items():
        np.testing.assert_allclose(got[name], w, atol=1e-10, rtol=1e-8, err_msg=name)


def test_philox_fixture():
    z = np.load(os.path.join(GOLD, 'philox_kat.npz'))
    got = ph.philox4x32_10(z['kat_in'][:, :4], z['kat_in'][:, 4:])
    assert (got == z['kat_out']).all()
    for site in range(4):
        assert (ph.random16(64, int(z['seed']), site) == z['fields'][site]).all()
