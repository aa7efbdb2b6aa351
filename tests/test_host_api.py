"""CPU-only checks of the host logic behind the C ABI: the library loads and
exports every symbol include/substation_amd.h declares, layout -> stride algebra
(pytorch_module/metahelpers.h:61-78), einsum -> GEMM classification
(pytorch_module/einsumparser.h:9-55) by brute force against numpy.einsum, the
host twin of the device mask generator against the oracle, configuration errors,
and the layouts schema.  No GPU call is made."""
import ctypes
import itertools
import os
import re

import numpy as np
import pytest

from oracle import philox_ref as ph
from substation_amd import _lib, layouts as L
from tests.einsums import EINSUMS, operand_layouts

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = '/root/reference/pytorch_module'


def _handle(B=2, S=4, H=3, E=6, lay=None, **kw):
    return _lib.Handle(_lib.make_config(B, S, H, E, lay or L.mi355x_layouts(), **kw))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    header = open(os.path.join(ROOT, 'include', 'substation_amd.h')).read()
    header = re.sub(r'/\*.*?\*/', '', header, flags=re.S)
    declared = set(re.findall(r'\b(?:void\*?|int|uint32_t|const char\*)\s+\*?(\w+)\s*\(', header))
    assert {'init', 'destroy', 'encoder_forward', 'encoder_backward'} <= declared
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    for name in declared:
        assert getattr(lib, name) is not None


def test_four_reference_exports_keep_their_pointer_counts():
    # pytorch_module/encoder.py:398-402
    assert len(_lib.SIGNATURES['encoder_forward'][1]) == 1 + 1 + 12 + 23 + 1
    assert len(_lib.SIGNATURES['encoder_backward'][1]) == 1 + 1 + 12 + 14 + (12 + 23 + 1) + 1


def test_layout_strides_match_numpy():
    h = _handle()
    sz = L.sizes_map(2, 4, 3, 6)
    for dims in ('BJI', 'HBJK', 'QPHBJ', 'IU', 'BJ'):
        for perm in itertools.permutations(dims):
            lay = ''.join(perm)
            a = np.empty(tuple(sz[d] for d in lay), dtype=np.float16)
            want = {d: s // 2 for d, s in zip(lay, a.strides)}
            got = h.strides(lay)
            for d in 'BJKHPIUQ':
                assert got[d] == want.get(d, 0), (lay, d)


def _emulate(info, A, B, shapeC):
    """Strided batched GEMM from the classifier's numbers only."""
    a, b = A.reshape(-1), B.reshape(-1)
    C = np.zeros(int(np.prod(shapeC)))
    K0, K1 = info['K0'], info['K1']
    k = np.arange(K0 * K1)
    ka = (k // K1) * info['sAK0'] + (k % K1) * info['sAK']
    kb = (k // K1) * info['sBK0'] + (k % K1) * info['sBK']
    for b0, b1, b2 in itertools.product(*(range(n) for n in info['nb'])):
        oa = b0 * info['sAb'][0] + b1 * info['sAb'][1] + b2 * info['sAb'][2]
        ob = b0 * info['sBb'][0] + b1 * info['sBb'][1] + b2 * info['sBb'][2]
        oc = b0 * info['sCb'][0] + b1 * info['sCb'][1] + b2 * info['sCb'][2]
        for m in range(info['M']):
            for n in range(info['N']):
                C[oc + m * info['sCM'] + n * info['sCN']] = np.dot(a[oa + m * info['sAM'] + ka],
                                                                  b[ob + n * info['sBN'] + kb])
    return C.reshape(shapeC)


@pytest.mark.parametrize('which', ['mi355x', 'bert-b8-l512-h16-e1024', 'bert-b96-l128-h16-e1024'])
def test_einsum_classification_brute_force(which):
    """Every contraction of the layer under three layout sets: the (batch, M, N, K,
    strides) the library derives reproduce numpy.einsum exactly."""
    lay = L.mi355x_layouts() if which == 'mi355x' else L.reference_layouts(which)
    B, S, H, E = 2, 3, 2, 4
    h = _handle(B, S, H, E, lay)
    sz = L.sizes_map(B, S, H, E)
    t = operand_layouts(lay)
    rng = np.random.default_rng(0)
    for name, a, b, c, _ in EINSUMS:
        la, lb, lc = t[a], t[b], t[c]
        A = rng.integers(-3, 4, size=tuple(sz[d] for d in la)).astype(np.float64)
        Bm = rng.integers(-3, 4, size=tuple(sz[d] for d in lb)).astype(np.float64)
        info = h.classify(la, lb, lc)
        want = np.einsum(f'{la},{lb}->{lc}'.lower(), A, Bm)
        got = _emulate(info, A, Bm, want.shape)
        assert info['batch'] * info['M'] * info['N'] == want.size, name
        np.testing.assert_array_equal(got, want, err_msg=f'{which}:{name} {la},{lb}->{lc}')


def test_einsum_random_permutations_either_work_or_fail_cleanly():
    B, S, H, E = 2, 3, 2, 4
    h = _handle(B, S, H, E)
    sz = L.sizes_map(B, S, H, E)
    rng = np.random.default_rng(1)
    ok = bad = 0
    for _ in range(150):
        la = ''.join(rng.permutation(list('PHBK')))
        lb = ''.join(rng.permutation(list('PHBJ')))
        lc = ''.join(rng.permutation(list('HBJK')))
        A = rng.integers(-3, 4, size=tuple(sz[d] for d in la)).astype(np.float64)
        Bm = rng.integers(-3, 4, size=tuple(sz[d] for d in lb)).astype(np.float64)
        try:
            info = h.classify(la, lb, lc)
        except _lib.SubstationError as e:
            assert 'einsum' in str(e)
            bad += 1
            continue
        want = np.einsum(f'{la},{lb}->{lc}'.lower(), A, Bm)
        np.testing.assert_array_equal(_emulate(info, A, Bm, want.shape), want)
        ok += 1
    assert ok > 50


def test_reference_8_case_table_is_covered():
    """The shipped configurations exercise both contiguity cases of A, B and C
    (pytorch_module/gemm.cuh:71-86)."""
    seen = set()
    for which in ('bert-b8-l512-h16-e1024', 'bert-b96-l128-h16-e1024'):
        lay = L.reference_layouts(which)
        h = _handle(8, 16, 2, 16, lay)
        t = operand_layouts(lay)
        for name, a, b, c, _ in EINSUMS:
            i = h.classify(t[a], t[b], t[c])
            assert i['sAM'] == 1 or i['sAK'] == 1, name       # gemm.cuh:59-61
            assert i['sBK'] == 1 or i['sBN'] == 1, name
            assert i['sCM'] == 1 or i['sCN'] == 1, name
            seen.add((i['sAM'] == 1, i['sBK'] == 1, i['sCM'] == 1))
    assert len(seen) >= 6


def test_host_philox_twin_matches_oracle():
    for seed, site, step, start, n in ((0x5EED, 0, 0, 0, 64), (0xDEADBEEFCAFE, 3, 7, 5, 1000),
                                       (1, 2, 2 ** 32 - 1, 2 ** 33 + 3, 100)):
        got = _lib.philox_fields_host(seed, site, step, start, n)
        want = ph.random16(n, seed, site, step, start=start)
        assert (got == want).all()
    lib = _lib.load()
    for p in (0.0, 0.1, 0.25, 0.5, 0.999, 1.0):
        assert lib.sub_dropout_threshold(p) == ph.threshold16(p)


def test_configuration_errors_are_reported_not_fatal():
    lay = L.mi355x_layouts()
    with pytest.raises(_lib.SubstationError, match='multiple of heads'):
        _handle(2, 4, 3, 8)
    bad = dict(lay); bad['forward_interm'] = [(n, ('QBJHP' if n != 'KKQQVV' else 'BQJHP')) if n == 'KKQQVV' else (n, l)
                                              for n, l in lay['forward_interm']]
    with pytest.raises(ValueError, match='must start with Q'):
        _lib.make_config(2, 4, 2, 8, bad)
    c = _lib.make_config(2, 4, 2, 8, lay)
    c.dtype = 1
    assert not _lib.load().init_cfg(ctypes.byref(c))
    assert b'fp16' in _lib.load().sub_last_error()
    c = _lib.make_config(2, 4, 2, 8, lay, p_softmax=1.5)
    assert not _lib.load().init_cfg(ctypes.byref(c))
    c = _lib.make_config(2, 4, 2, 8, lay)
    c.abi_version = 99
    assert not _lib.load().init_cfg(ctypes.byref(c))
    # an unconfigured handle refuses to run
    lib = _lib.load()
    h = lib.init()
    arr = (ctypes.c_void_p * 37)(*([1] * 37))
    assert lib.sub_encoder_forward(h, arr, 37) < 0 and b'not configured' in lib.sub_last_error()
    assert lib.sub_encoder_forward(h, arr, 36) < 0
    lib.destroy(h)


def test_layouts_schema_roundtrip(tmp_path):
    for lay in (L.mi355x_layouts(), L.reference_layouts('bert-b8-l512-h16-e1024'),
                L.reference_layouts('bert-b96-l128-h16-e1024')):
        L.validate(lay)
        assert [n for n, _ in lay['params']] == L.PARAM_NAMES
        assert [n for n, _ in lay['forward_interm']] == L.FWD_NAMES
        assert [n for n, _ in lay['backward_interm']] == L.BWD_NAMES
        p = tmp_path / 'l.pickle'
        L.save_layouts(lay, str(p))
        assert L.load_layouts(str(p)) == lay
    with pytest.raises(ValueError):
        L.validate({'input': ('X', 'BJI')})
    # a pickle that refers to any class or function is refused
    import pickle
    evil = tmp_path / 'evil.pickle'
    evil.write_bytes(pickle.dumps(os.getcwd))
    with pytest.raises(pickle.UnpicklingError):
        L.load_layouts(str(evil))


@pytest.mark.skipif(not os.path.isdir(REF), reason='reference checkout not mounted')
@pytest.mark.parametrize('name', ['bert-b8-l512-h16-e1024', 'bert-b96-l128-h16-e1024'])
def test_reference_layout_literals_equal_the_shipped_pickles(name):
    """The literals in substation_amd/layouts.py against the reference's data
    files, read with the data-only unpickler (nothing from the file executes)."""
    got = L.load_layouts(os.path.join(REF, f'layouts-{name}.pickle'))
    want = L.reference_layouts(name)
    for key in ('input', 'output', 'params', 'forward_interm', 'backward_interm'):
        assert [tuple(x) for x in got[key]] == [tuple(x) for x in want[key]] or tuple(got[key]) == tuple(want[key]), key
    assert got['special_dims'] == want['special_dims']
    assert got['algorithms'] == want['algorithms']


def test_einsum_with_addend_rejects_an_addend_that_is_no_sub_block_of_the_output():
    """sub_op_einsum_add checks the addend's layout on the host, before any launch:
    its dims must be free or batch dims of the output, each merged group in one
    dense run (the argument check of an epilogue addend; no GPU needed to fail)."""
    h = _handle(2, 128, 2, 128)
    lib = _lib.load()
    one = ctypes.c_void_p(16)
    s = lambda t: t.encode()
    # U is not a dim of the output
    rc = lib.sub_op_einsum_add(h.ptr, one, s('BJI'), one, s('HPI'), one, s('U'), one, s('BJHP'), 1.0)
    assert rc < 0 and b'sub_op_einsum_add' in lib.sub_last_error()
    # (H, P) merged in the output but transposed in the addend: not one stride
    rc = lib.sub_op_einsum_add(h.ptr, one, s('BJI'), one, s('HPI'), one, s('PH'), one, s('BJHP'), 1.0)
    assert rc < 0 and b'sub_op_einsum_add' in lib.sub_last_error()
    # a null addend
    rc = lib.sub_op_einsum_add(h.ptr, one, s('BJI'), one, s('HPI'), None, s('HP'), one, s('BJHP'), 1.0)
    assert rc < 0 and b'null addend' in lib.sub_last_error()
