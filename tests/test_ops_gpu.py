"""GPU parity of every fused operator against the oracle's closed forms
(oracle/encoder_ref.py op_*, restating pytorch_module/benchmark.py), through the
C ABI.  Inputs are rounded to fp16 first, so the only difference left is the
device's fp32-internal arithmetic and one fp16 rounding per output: tolerance
1e-2 relative (pytorch_module/benchmark.py:294-302 uses atol=rtol=1e-2).
Dropout masks are compared bit-exactly with oracle/philox_ref.py."""
import itertools

import numpy as np
import pytest
import torch

from oracle import encoder_ref as ref
from oracle import philox_ref as ph
from tests.helpers import assert_close, from_layout, h16, to_layout

pytestmark = pytest.mark.gpu

SEED = 0x5EED


def _ops(B, L, H, E, act='relu', U=None):
    from substation_amd.ops import Ops
    o = Ops(B, L, H, E, activation=act, seed=SEED, intermediate_size=U)
    return o


def _perms(canon, keep=None, limit=4):
    """A few layouts of `canon`: the canonical one plus others (deterministic)."""
    allp = [''.join(p) for p in itertools.permutations(canon)]
    picks = [canon, allp[-1]] + allp[1:len(allp) - 1:max(1, len(allp) // limit)]
    out = []
    for p in picks:
        if p not in out:
            out.append(p)
    return out[:limit + 1]


SIZES = [(2, 16, 2, 32), (3, 24, 2, 48), (2, 128, 4, 512)]


# the last four: short rows, several side by side in a wave (needs >= 16384 rows)
@pytest.mark.parametrize('B,L,H,E', SIZES + [(1, 520, 1, 8), (8, 128, 16, 64), (4, 256, 16, 64),
                                            (9, 120, 16, 32), (6, 200, 16, 32),
                                            (1, 2048, 2, 16)])     # rows of 2048 keys: four packs per lane
@pytest.mark.parametrize('p', [0.0, 0.5])
def test_softmax_and_backward(B, L, H, E, p):
    o = _ops(B, L, H, E)
    rng = np.random.default_rng(1)
    beta = h16(rng.normal(size=(H, B, L, L)) * 2)
    ddrop = h16(rng.normal(size=(H, B, L, L)))
    scale = 0.125
    want_mask = ph.dropout_mask((H, B, L, L), p, SEED, ph.SITE_SOFTMAX, step=3)
    alpha_w, drop_w = ref.op_softmax(beta, want_mask, scale)
    for lin, lout in (('HBJK', 'HBJK'), ('BHJK', 'BHJK'), ('HBJK', 'JBHK'), ('KJBH', 'HBKJ')):
        o.set_rng(SEED, 3)
        t_beta = to_layout(beta, 'HBJK', lin)
        a, m, d = o.empty(lout), o.empty(lout), o.empty(lin)
        o.softmax(t_beta, lin, a, lout, m, lout, d, lin, scale=scale, p=p, site=0)
        torch.cuda.synchronize()
        got_mask = from_layout(m, 'HBJK', lout)
        assert (got_mask == want_mask).all(), 'mask differs from the oracle'
        assert_close(from_layout(a, 'HBJK', lout), alpha_w, name='ALPHA ' + lin)
        assert_close(from_layout(d, 'HBJK', lin), drop_w, name='ATTN_DROP ' + lin)
        # ATTN_DROP is exactly ALPHA * MASK in fp16
        assert (from_layout(d, 'HBJK', lin) == from_layout(a, 'HBJK', lout) * got_mask).all()
        # backward on the device's own fp16 alpha
        alpha16 = from_layout(a, 'HBJK', lout)
        dbeta = o.empty(lout)
        o.bs(a, lout, m, lout, to_layout(ddrop, 'HBJK', lin), lin, dbeta, lout, scale=scale)
        torch.cuda.synchronize()
        assert_close(from_layout(dbeta, 'HBJK', lout), ref.op_bs(alpha16, want_mask, ddrop, scale),
                     name='DBETA ' + lin)


def test_softmax_baseline_config_full_size():
    """BASELINE configs[1]: scores [H=16,B=8,J=512,K=512] ~ N(0,1), scale 1/sqrt(64),
    p=0.1 seeded, forward plus softmax backward with dY ~ N(0,1), at full size."""
    B, L, H, E = 8, 512, 16, 1024
    o = _ops(B, L, H, E)
    rng = np.random.default_rng(1002)
    beta = h16(rng.normal(size=(H, B, L, L)))
    ddrop = h16(rng.normal(size=(H, B, L, L)))
    scale, p, lay = 0.125, 0.1, 'HBJK'
    want_mask = ph.dropout_mask((H, B, L, L), p, SEED, ph.SITE_SOFTMAX, step=0)
    o.set_rng(SEED, 0)
    a, m, d, db = o.empty(lay), o.empty(lay), o.empty(lay), o.empty(lay)
    o.softmax(to_layout(beta, lay, lay), lay, a, lay, m, lay, d, lay, scale=scale, p=p, site=0)
    o.bs(a, lay, m, lay, to_layout(ddrop, lay, lay), lay, db, lay, scale=scale)
    torch.cuda.synchronize()
    alpha_w, drop_w = ref.op_softmax(beta, want_mask, scale)
    alpha16 = from_layout(a, lay, lay)
    assert (from_layout(m, lay, lay) == want_mask).all()
    assert 0.099 < 1 - want_mask.mean() < 0.101
    assert_close(alpha16, alpha_w, name='ALPHA')
    assert (from_layout(d, lay, lay) == alpha16 * want_mask).all()
    assert_close(from_layout(db, lay, lay), ref.op_bs(alpha16, want_mask, ddrop, scale), name='DBETA')
    assert np.abs(alpha16.sum(axis=-1) - 1).max() < 4e-3


@pytest.mark.parametrize('B,L,H,E', [(2, 16, 2, 32), (2, 128, 4, 512), (8, 128, 16, 64), (3, 40, 2, 16),
                                     (1, 2048, 2, 16)])
def test_softmax_with_attention_mask(B, L, H, E):
    """alpha = softmax(scale * beta + mask_scale * attn_mask) with a causal mask
    plus finite entries, in both mask layouts; the backward operator needs no mask."""
    o = _ops(B, L, H, E)
    rng = np.random.default_rng(2)
    beta = h16(rng.normal(size=(H, B, L, L)) * 2)
    am = h16(np.triu(np.full((L, L), -np.inf), k=1) + np.tril(rng.normal(size=(L, L))))
    scale, mscale, p = 0.25, 0.5, 0.3
    want_mask = ph.dropout_mask((H, B, L, L), p, SEED, ph.SITE_SOFTMAX, step=1)
    x = scale * beta + mscale * am[None, None]
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    alpha_w = e / e.sum(axis=-1, keepdims=True)
    for lay, lam in (('HBJK', 'JK'), ('BHJK', 'KJ'), ('JBHK', 'JK')):
        o.set_rng(SEED, 1)
        a, m, d = o.empty(lay), o.empty(lay), o.empty(lay)
        t_am = torch.from_numpy(am if lam == 'JK' else am.T.copy()).half().cuda()
        o.softmax(to_layout(beta, 'HBJK', lay), lay, a, lay, m, lay, d, lay, scale=scale, p=p, site=0,
                  attn_mask=t_am, l_attn_mask=lam, mask_scale=mscale)
        torch.cuda.synchronize()
        got = from_layout(a, 'HBJK', lay)
        assert (from_layout(m, 'HBJK', lay) == want_mask).all()
        assert (got[..., np.triu_indices(L, 1)[0], np.triu_indices(L, 1)[1]] == 0).all()   # future positions
        assert_close(got, alpha_w, name='ALPHA masked ' + lay)
        assert (from_layout(d, 'HBJK', lay) == got * want_mask).all()


# (rows of 1000 and 776 features: the last pack of a lane's two lies outside the row for some lanes;
# 66000 rows of 64: more rows than the launch has waves, a wave takes several)
@pytest.mark.parametrize('B,L,H,E', SIZES + [(2, 8, 1, 1024), (1, 4, 1, 4096), (2, 3, 1, 20), (3, 40, 1, 1000),
                                            (2, 130, 1, 776), (66, 1000, 1, 64)])
@pytest.mark.parametrize('p', [0.0, 0.3])
def test_bdrln_and_blnrd(B, L, H, E, p):
    o = _ops(B, L, H, E)
    rng = np.random.default_rng(2)
    inp = h16(rng.normal(size=(B, L, E))); resid = h16(rng.normal(size=(B, L, E)))
    lb = h16(rng.normal(size=E) * 0.1); s = h16(1 + 0.1 * rng.normal(size=E)); b = h16(0.1 * rng.normal(size=E))
    dout = h16(rng.normal(size=(B, L, E)))
    want_mask = ph.dropout_mask((B, L, E), p, SEED, ph.SITE_RESID1, step=0)
    for lay, lay2, lstd in (('BJI', 'BJI', 'BJ'), ('JBI', 'BJI', 'JB'), ('IBJ', 'JBI', 'BJ')):
        o.set_rng(SEED, 0)
        t_in = to_layout(inp, 'BJI', lay)
        lin = t_in if lay == 'BJI' else o.empty(lay)          # in-place bias add as in the layer
        mask, diff, normed, out, istd = o.empty(lay2), o.empty(lay2), o.empty(lay), o.empty(lay), o.empty(lstd)
        dev = lambda v: torch.from_numpy(v).to(torch.float16).cuda()
        o.bdrln(t_in, lay, to_layout(resid, 'BJI', lay2), lay2, dev(lb), dev(s), dev(b), lin, lay,
                mask, lay2, diff, lay2, normed, lay, out, lay, istd, lstd, p=p, site=1)
        torch.cuda.synchronize()
        assert (from_layout(mask, 'BJI', lay2) == want_mask).all()
        lin_w = h16(inp + lb)               # the device rounds LIN before using it
        _, istd_w, diff_w, normed_w, out_w = ref.op_bdrln(lin_w, resid, 0.0, s, b, want_mask)
        assert (from_layout(lin, 'BJI', lay) == lin_w).all()
        assert_close(from_layout(istd, 'BJ', lstd), istd_w, name='ISTD')
        assert_close(from_layout(diff, 'BJI', lay2), diff_w, name='DIFF')
        assert_close(from_layout(normed, 'BJI', lay), normed_w, name='NORMED')
        assert_close(from_layout(out, 'BJI', lay), out_w, name='OUT')
        # backward from the device's own fp16 DIFF / ISTD
        d1, d2 = o.empty(lay), o.empty(lay2)
        o.blnrd(to_layout(dout, 'BJI', lay2), lay2, istd, lstd, diff, lay2, mask, lay2, d1, lay, d2, lay2)
        torch.cuda.synchronize()
        w1, w2 = ref.op_blnrd(dout, from_layout(istd, 'BJ', lstd), from_layout(diff, 'BJI', lay2), want_mask)
        assert_close(from_layout(d1, 'BJI', lay), w1, name='D_LN_IN')
        assert_close(from_layout(d2, 'BJI', lay2), w2, name='D_DROP_IN')


@pytest.mark.parametrize('B,L,H,E', SIZES + [(2, 5, 1, 8)])
@pytest.mark.parametrize('act', ['relu', 'gelu'])
def test_bad_and_bdrlb(B, L, H, E, act):
    U = 4 * E if E != 8 else 20
    o = _ops(B, L, H, E, act, U=U)
    rng = np.random.default_rng(3)
    inp = h16(rng.normal(size=(B, L, U))); bias = h16(rng.normal(size=U) * 0.5)
    ddrop = h16(rng.normal(size=(B, L, U)))
    p = 0.25
    want_mask = ph.dropout_mask((B, L, U), p, SEED, ph.SITE_ACT, step=1)
    dev = lambda v: torch.from_numpy(v).to(torch.float16).cuda()
    for lay, lay2 in (('BJU', 'BJU'), ('UBJ', 'BJU'), ('JBU', 'JUB')):
        o.set_rng(SEED, 1)
        lin, mask, out = o.empty(lay2), o.empty(lay), o.empty(lay2)
        o.bad(to_layout(inp, 'BJU', lay), lay, dev(bias), lin, lay2, mask, lay, out, lay2, p=p, site=2)
        torch.cuda.synchronize()
        assert (from_layout(mask, 'BJU', lay) == want_mask).all()
        lin_w = h16(inp + bias)
        assert (from_layout(lin, 'BJU', lay2) == lin_w).all()
        assert_close(from_layout(out, 'BJU', lay2), ref.op_bad(lin_w, 0.0, want_mask, act)[1], name='DROP2')
        dlin, dbias = o.empty(lay), torch.empty(U, dtype=torch.float16, device='cuda')
        o.bdrlb(to_layout(ddrop, 'BJU', lay2), lay2, mask, lay, lin, lay2, dlin, lay, dbias)
        torch.cuda.synchronize()
        w_dlin, w_dbias = ref.op_bdrlb(ddrop, want_mask, lin_w, act)
        assert_close(from_layout(dlin, 'BJU', lay), w_dlin, name='DLIN1')
        assert_close(dbias.float().cpu().numpy(), w_dbias, name='DLINB1')


def test_deferred_column_sums_give_the_same_bits():
    """sub_ops_defer: between the two calls the column sums of the operators (here
    nine of them: more than the list of six holds, so it is finished early once,
    and the scratch buffer has to start over as well) are finished by shared
    launches; every gradient vector must equal, bit for bit, what the operator gives
    when it finishes its sums itself, and must be complete once the block ends."""
    B, L, H, E = 4, 256, 4, 512
    o = _ops(B, L, H, E)
    rng = np.random.default_rng(9)
    dev = lambda v: torch.from_numpy(h16(v)).to(torch.float16).cuda()
    scale = dev(1 + 0.1 * rng.normal(size=E))
    tensors = [(dev(rng.normal(size=(B, L, E))), dev(rng.normal(size=(B, L, E)))) for _ in range(3)]
    vec = lambda: torch.zeros(E, dtype=torch.float16, device='cuda')

    def run():
        outs = []
        for inp, dout in tensors:
            din, ds, db, dbo = o.empty('BJI'), vec(), vec(), vec()
            o.bsb(inp, 'BJI', scale, dout, 'BJI', din, 'BJI', ds, db)
            o.baob(dout, 'BJI', dbo)
            dl = vec()
            din2, ds2, db2 = o.empty('BJI'), vec(), vec()
            o.ebsb(inp, 'BJI', scale, dout, 'BJI', inp, 'BJI', dout, 'BJI', din2, 'BJI', ds2, db2, dl)
            outs += [din, ds, db, dbo, din2, ds2, db2, dl]
        return outs

    plain = run()
    torch.cuda.synchronize()
    for _ in range(3):                  # the scratch buffer grows to hold a whole block within a few blocks
        with o.deferred_column_sums():
            deferred = run()
    torch.cuda.synchronize()
    for a, b in zip(plain, deferred):
        assert float(a.float().abs().max()) > 0
        assert torch.equal(a, b)
    # the handle is back to finishing every reduction in its own call
    dbo = vec()
    o.baob(tensors[0][1], 'BJI', dbo)
    torch.cuda.synchronize()
    assert torch.equal(dbo, plain[3])


@pytest.mark.parametrize('B,L,H,E', SIZES + [(2, 3, 1, 20), (4, 64, 1, 1024), (2, 8, 1, 4096)])
def test_bsb_ebsb_baob_bei(B, L, H, E):
    o = _ops(B, L, H, E)
    rng = np.random.default_rng(4)
    g = lambda: h16(rng.normal(size=(B, L, E)))
    inp, dout, d2, dl = g(), g(), g(), g()
    s = h16(1 + 0.1 * rng.normal(size=E))
    dev = lambda v: torch.from_numpy(v).to(torch.float16).cuda()
    vec = lambda: torch.empty(E, dtype=torch.float16, device='cuda')
    for lay, lay2 in (('BJI', 'BJI'), ('IBJ', 'JBI'), ('JBI', 'BJI')):
        din, ds, db = o.empty(lay2), vec(), vec()
        o.bsb(to_layout(inp, 'BJI', lay), lay, dev(s), to_layout(dout, 'BJI', lay2), lay2, din, lay2, ds, db)
        torch.cuda.synchronize()
        w = ref.op_bsb(inp, s, dout)
        assert_close(from_layout(din, 'BJI', lay2), w[0], name='DLN2')
        assert_close(ds.float().cpu().numpy(), w[1], name='DS2')
        assert_close(db.float().cpu().numpy(), w[2], name='DB2')
        din, ds, db, dlb = o.empty(lay), vec(), vec(), vec()
        o.ebsb(to_layout(inp, 'BJI', lay), lay, dev(s), to_layout(dout, 'BJI', lay2), lay2,
               to_layout(d2, 'BJI', lay), lay, to_layout(dl, 'BJI', lay2), lay2, din, lay, ds, db, dlb)
        torch.cuda.synchronize()
        w = ref.op_ebsb(inp, s, dout, d2, dl)
        assert_close(from_layout(din, 'BJI', lay), w[0], name='DLN1')
        assert_close(ds.float().cpu().numpy(), w[1], name='DS1')
        assert_close(db.float().cpu().numpy(), w[2], name='DB1')
        assert_close(dlb.float().cpu().numpy(), w[3], name='DLINB2')
        dbo = vec()
        o.baob(to_layout(dout, 'BJI', lay), lay, dbo)
        dx = o.empty(lay2)
        o.bei(to_layout(inp, 'BJI', lay), lay, to_layout(d2, 'BJI', lay2), lay2, dx, lay2)
        torch.cuda.synchronize()
        assert_close(dbo.float().cpu().numpy(), ref.op_baob(dout), name='DBO')
        assert_close(from_layout(dx, 'BJI', lay2), ref.op_bei(inp, d2), name='DX')


@pytest.mark.parametrize('B,L,H,E', SIZES)
def test_aib_baib(B, L, H, E):
    o = _ops(B, L, H, E)
    P = E // H
    rng = np.random.default_rng(5)
    w = h16(rng.normal(size=(3, P, H, B, L))); bias = h16(rng.normal(size=(3, P, H)))
    for lin, lout, lb in (('QPHBJ', 'QPHBJ', 'QPH'), ('QPHBJ', 'QHBPJ', 'QPH'), ('QBJHP', 'QBJHP', 'QHP'),
                          ('QJBPH', 'QBHJP', 'QHP')):
        out = o.empty(lout)
        o.aib(to_layout(w, 'QPHBJ', lin), lin, to_layout(bias, 'QPH', lb), lb, out, lout)
        db = o.empty(lb)
        o.baib(to_layout(w, 'QPHBJ', lin), lin, db, lb)
        torch.cuda.synchronize()
        assert_close(from_layout(out, 'QPHBJ', lout), ref.op_aib(w, bias), name='KKQQVV ' + lin)
        assert_close(from_layout(db, 'QPH', lb), ref.op_baib(w), name='DBKQV ' + lin)


@pytest.mark.parametrize('B,H,P,J,K,p,masked,l_q,l_kv', [
    (2, 2, 64, 128, 128, 0.1, False, 'BJHP', 'BKHP'),
    (2, 2, 64, 128, 384, 0.1, False, 'BJHP', 'BKHP'),      # more keys than queries (encoder-decoder attention)
    (1, 3, 64, 256, 128, 0.0, False, 'BHJP', 'BHKP'),      # fewer keys than queries, head-major rows
    (2, 2, 128, 128, 256, 0.25, True, 'JBHP', 'KBHP'),     # head size 128, additive mask, position-major rows
    (8, 16, 64, 512, 512, 0.1, False, 'BJHP', 'BKHP'),     # the bench workload's attention
    (1, 2, 128, 2048, 2048, 0.1, True, 'BJHP', 'BKHP'),    # 64 key tiles, head size 128 (the wide workload's shape per head)
])
def test_attention_operator_forward_and_backward(B, H, P, J, K, p, masked, l_q, l_kv):
    """The attention kernels as one operator against the closed form
    (substation/attention.py:31-179 restated for one head: softmax over the keys of
    scale*(q.k^T + mask), {0,1} dropout mask without rescale, weighted sum of v,
    and its gradients), in float64 on the fp16-rounded inputs.  The keep bits are
    compared exactly with the oracle's Philox stream over the [H,B,J,K] index."""
    o = _ops(B, 128, H, H * P)
    o.set_rng(SEED, 2)
    rng = np.random.default_rng(J * 7 + K)
    q = h16(rng.standard_normal((B, J, H, P)))
    k = h16(rng.standard_normal((B, K, H, P)))
    v = h16(rng.standard_normal((B, K, H, P)))
    d_out = h16(rng.standard_normal((B, J, H, P)))
    scale = 1.0 / np.sqrt(P)
    am = None
    if masked:
        am = h16(rng.standard_normal((J, K)))
        am[np.triu_indices(J, 1, K)] = -np.inf
        am[:, 0] = 0.0                                       # no row is masked out entirely
    tq, tk, tv = to_layout(q, 'BJHP', l_q), to_layout(k, 'BKHP', l_kv), to_layout(v, 'BKHP', l_kv)
    tdo = to_layout(d_out, 'BJHP', l_q)
    out, dq = torch.empty_like(tq), torch.empty_like(tq)
    dk, dv = torch.empty_like(tk), torch.empty_like(tk)
    stats, keep = o.attention_workspace(J, K)
    tam = None if am is None else torch.from_numpy(am).half().cuda()
    o.attention_forward(tq, l_q, tk, tv, l_kv, out, l_q, stats, keep, scale, p=p, site=ph.SITE_SOFTMAX, attn_mask=tam)
    o.attention_backward(tq, l_q, tk, tv, l_kv, out, l_q, tdo, l_q, stats, keep, dq, l_q, dk, dv, l_kv, scale,
                         attn_mask=tam)
    torch.cuda.synchronize()

    mask = ph.dropout_mask((H, B, J, K), p, SEED, ph.SITE_SOFTMAX, step=2, dtype=np.float64)
    words = keep.cpu().numpy().view(np.uint32).reshape(H, B, J, K // 32)
    bits = ((words[..., None] >> np.arange(32, dtype=np.uint32)) & 1).reshape(H, B, J, K)
    assert np.array_equal(bits, mask.astype(np.uint32))

    s = np.einsum('bjhp,bkhp->hbjk', q, k)
    if am is not None:
        s = s + am
    s = s * scale
    e = np.exp(s - s.max(-1, keepdims=True))
    alpha = e / e.sum(-1, keepdims=True)
    drop = alpha * mask
    want_out = np.einsum('hbjk,bkhp->bjhp', drop, v)
    d_drop = np.einsum('bjhp,bkhp->hbjk', d_out, v)
    d_alpha = d_drop * mask
    d_s = alpha * (d_alpha - (alpha * d_alpha).sum(-1, keepdims=True))
    want_dq = scale * np.einsum('hbjk,bkhp->bjhp', d_s, k)
    want_dk = scale * np.einsum('hbjk,bjhp->bkhp', d_s, q)
    want_dv = np.einsum('hbjk,bjhp->bkhp', drop, d_out)
    lse = stats.cpu().numpy()[:H * B * J].reshape(H, B, J)
    want_lse = (s.max(-1) + np.log(e.sum(-1))) / np.log(2.0)
    assert_close(lse, want_lse, tol=1e-3, name='log-sum-exp')
    assert_close(from_layout(out, 'BJHP', l_q), want_out, name='out')
    assert_close(from_layout(dq, 'BJHP', l_q), want_dq, name='dq')
    assert_close(from_layout(dk, 'BKHP', l_kv), want_dk, name='dk')
    assert_close(from_layout(dv, 'BKHP', l_kv), want_dv, name='dv')


# (1000, 776: rows that end inside a lane's second pack; 5000 rows of 64: more rows than the launch has waves;
# 2048, 3000, 4096 features: a row shared by two or four waves -- 150 and 1200 rows make several passes with a
# last one that leaves waves without a row, 3000 leaves the fourth wave of a row without features)
@pytest.mark.parametrize('B,L,H,E', [(2, 128, 4, 512), (4, 64, 1, 1024), (3, 24, 2, 48), (1, 4, 1, 4096),
                                     (3, 40, 1, 1000), (2, 130, 1, 776), (5, 1000, 1, 64),
                                     (3, 50, 1, 2048), (2, 70, 1, 3000), (4, 300, 1, 4096)])
@pytest.mark.parametrize('extended', [False, True])
def test_ln_backward_one_launch_or_separate(B, L, H, E, extended):
    """sub_op_ln_backward (bsb + blnrd, or ebsb + blnrd + baob) against the oracle's
    operators, for sizes and layouts the one-launch kernel takes (rows of up to 1024
    contiguous features, of up to 4096 in its plain form) and for ones it hands to the
    separate operators."""
    o = _ops(B, L, H, E)
    rng = np.random.default_rng(12)
    g = lambda: h16(rng.normal(size=(B, L, E)))
    normed, d1, d2, dl, diff = g(), g(), g(), g(), g()
    istd = h16(1.0 + 0.2 * rng.random(size=(B, L)))
    s = h16(1 + 0.1 * rng.normal(size=E))
    mask = ph.dropout_mask((B, L, E), 0.3, SEED, ph.SITE_RESID1, step=0)
    dev = lambda v: torch.from_numpy(np.asarray(v)).to(torch.float16).cuda()
    vec = lambda: torch.empty(E, dtype=torch.float16, device='cuda')
    for lay, lay2, lstd in (('BJI', 'BJI', 'BJ'), ('JBI', 'BJI', 'JB'), ('IBJ', 'JBI', 'BJ')):
        gt, o1, o2 = o.empty(lay), o.empty(lay2), o.empty(lay)
        ds, db, dlb, dob = vec(), vec(), vec(), vec()
        kw = {}
        if extended:
            kw = dict(dout2=to_layout(d2, 'BJI', lay2), l_dout2=lay2, dlinear=to_layout(dl, 'BJI', lay), l_dlinear=lay,
                      dlinear_bias=dlb, dout_bias=dob)
        o.ln_backward(to_layout(normed, 'BJI', lay), lay, dev(s), to_layout(d1, 'BJI', lay2), lay2,
                      to_layout(istd, 'BJ', lstd), lstd, to_layout(diff, 'BJI', lay2), lay2,
                      to_layout(mask, 'BJI', lay), lay, gt, lay, o1, lay2, o2, lay, ds, db, **kw)
        torch.cuda.synchronize()
        if extended:
            w = ref.op_ebsb(normed, s, d1, d2, dl)
        else:
            w = ref.op_bsb(normed, s, d1)
        assert_close(from_layout(gt, 'BJI', lay), w[0], name='G')
        assert_close(ds.float().cpu().numpy(), w[1], name='DSCALE')
        assert_close(db.float().cpu().numpy(), w[2], name='DBIAS')
        w1, w2 = ref.op_blnrd(from_layout(gt, 'BJI', lay), istd, diff, mask)      # from the device's rounded G
        assert_close(from_layout(o1, 'BJI', lay2), w1, name='D_LN_IN')
        assert_close(from_layout(o2, 'BJI', lay), w2, name='D_DROP_IN')
        if extended:
            assert_close(dlb.float().cpu().numpy(), w[3], name='DLINEAR_BIAS')
            assert_close(dob.float().cpu().numpy(), ref.op_baob(from_layout(o2, 'BJI', lay)), name='DOUT_BIAS')


@pytest.mark.parametrize('dims', [(2, 64, 2, 128), (3, 40, 3, 120), (2, 5, 1, 20), (8, 512, 16, 1024)])
def test_relayout_is_a_permutation_of_the_same_tensor(dims):
    """sub_op_relayout against a permuted copy, bit for bit: tiled transposes (the contiguous dim changes),
    vector copies (it stays), the scalar path (sizes that are not multiples of 8), five dims."""
    B, L, H, E = dims
    o = _ops(B, L, H, E)
    g = torch.Generator(device='cuda').manual_seed(11)
    cases = [('BJI', 'IBJ'), ('IBJ', 'BJI'), ('JBI', 'BJI'), ('BJU', 'UBJ'), ('QPHBJ', 'QBJHP'), ('QBJHP', 'QPHBJ'),
             ('QPHI', 'QHPI'), ('IPH', 'IHP'), ('UI', 'IU'), ('HBJK', 'KJBH')]
    if B * L * E > 1 << 20:
        cases = cases[:5]
    for l_src, l_dst in cases:
        src = o.empty(l_src).normal_(0.0, 1.0, generator=g)
        dst = o.empty(l_dst).fill_(float('nan'))
        o.relayout(src, l_src, dst, l_dst)
        torch.cuda.synchronize()
        want = src.permute([l_src.index(d) for d in l_dst]).contiguous()
        assert torch.equal(dst, want), (dims, l_src, l_dst)
