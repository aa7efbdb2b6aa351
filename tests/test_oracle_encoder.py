"""Pins oracle/encoder_ref.py against stock PyTorch, the way the reference's own
test/test_transformer_torch.py does (weight mapping at :129-141, :231-296), and
against autograd of the device-path graph with explicit mask nodes."""
import numpy as np
import pytest
import scipy.special
import torch
import torch.nn.functional as F

from oracle import encoder_ref as ref
from tests import torch_graph as tg

B, L, H, E = 3, 7, 4, 8   # test/test_transformer_torch.py:13-27 defaults


def _np(d):
    return {k: v.numpy() for k, v in d.items()}


@pytest.mark.parametrize('activation', ['relu', 'gelu'])
@pytest.mark.parametrize('masked', [False, True])
def test_encoder_matches_torch_transformer_layer(activation, masked):
    params, X, DY = tg.make_inputs(B, L, H, E, seed=11, w_std=0.3, b_std=0.3)
    a = ref.module_params_to_numpy(_np(params))
    P = E // H
    act = 'relu' if activation == 'relu' else tg.gelu_tanh
    layer = torch.nn.TransformerEncoderLayer(E, H, 4 * E, dropout=0.0, activation=act,
                                             batch_first=True, norm_first=False).double()
    with torch.no_grad():
        mha = layer.self_attn
        mha.in_proj_weight.copy_(torch.from_numpy(np.concatenate(
            [a['attn_wq'].reshape(H * P, E), a['attn_wk'].reshape(H * P, E),
             a['attn_wv'].reshape(H * P, E)])))
        mha.in_proj_bias.copy_(torch.from_numpy(a['attn_in_b'].reshape(-1)))
        mha.out_proj.weight.copy_(torch.from_numpy(a['attn_wo']))
        mha.out_proj.bias.copy_(torch.from_numpy(a['attn_out_b']))
        layer.linear1.weight.copy_(torch.from_numpy(a['linear1_w']))
        layer.linear1.bias.copy_(torch.from_numpy(a['linear1_b']))
        layer.linear2.weight.copy_(torch.from_numpy(a['linear2_w']))
        layer.linear2.bias.copy_(torch.from_numpy(a['linear2_b']))
        layer.norm1.weight.copy_(params['S1']); layer.norm1.bias.copy_(params['B1'])
        layer.norm2.weight.copy_(params['S2']); layer.norm2.bias.copy_(params['B2'])
    x = X.clone().requires_grad_(True)
    layer.train()
    scale = 1.0 / np.sqrt(P)
    attn_mask = None
    if masked:
        # causal, plus finite entries below the diagonal so that the place where the
        # mask enters (raw scores, before the scaling: attention.py:65-68) is pinned;
        # torch adds its mask after the scaling
        rng = np.random.default_rng(5)
        attn_mask = ref.gen_attn_mask(L, L) + np.tril(rng.normal(size=(L, L)))
        y = layer(x, src_mask=torch.from_numpy(scale * attn_mask))
    else:
        y = layer(x)
    y.backward(DY)

    f = ref.encoder(X.numpy(), a['attn_wq'], a['attn_wk'], a['attn_wv'], a['attn_wo'],
                    a['attn_in_b'], a['attn_out_b'], scale, a['norm1_scale'], a['norm1_bias'],
                    a['norm2_scale'], a['norm2_bias'], a['linear1_w'], a['linear1_b'],
                    a['linear2_w'], a['linear2_b'], activation=activation, attn_mask=attn_mask)
    g = ref.encoder_backward(X.numpy(), DY.numpy(), f, a['attn_wq'], a['attn_wk'], a['attn_wv'],
                             a['attn_wo'], scale, a['norm1_scale'], a['norm2_scale'],
                             a['linear1_w'], a['linear1_b'], a['linear2_w'], a['linear2_b'],
                             activation=activation)
    tol = dict(atol=1e-10, rtol=1e-9)
    np.testing.assert_allclose(f['y'], y.detach().numpy(), **tol)
    np.testing.assert_allclose(g['dx'], x.grad.numpy(), **tol)
    dw_in = mha.in_proj_weight.grad.numpy().reshape(3, H, P, E)
    np.testing.assert_allclose(g['dattn_wq'], dw_in[0], **tol)
    np.testing.assert_allclose(g['dattn_wk'], dw_in[1], **tol)
    np.testing.assert_allclose(g['dattn_wv'], dw_in[2], **tol)
    np.testing.assert_allclose(g['dattn_in_b'].reshape(-1), mha.in_proj_bias.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dattn_wo'], mha.out_proj.weight.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dattn_out_b'], mha.out_proj.bias.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dlinear1_w'], layer.linear1.weight.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dlinear1_b'], layer.linear1.bias.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dlinear2_w'], layer.linear2.weight.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dlinear2_b'], layer.linear2.bias.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dnorm1_scale'], layer.norm1.weight.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dnorm1_bias'], layer.norm1.bias.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dnorm2_scale'], layer.norm2.weight.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dnorm2_bias'], layer.norm2.bias.grad.numpy(), **tol)


@pytest.mark.parametrize('activation,pdrop', [('relu', 0.0), ('relu', 0.3), ('gelu', 0.3)])
def test_run_named_matches_autograd_of_device_graph(activation, pdrop):
    """All four dropout sites, every named intermediate, DX and the 12 gradients."""
    params, X, DY = tg.make_inputs(2, 6, 2, 8, seed=5, w_std=0.4, b_std=0.2)
    masks = tg.make_masks(2, 6, 2, 8, pdrop, seed=5) if pdrop else None
    want = tg.run(params, X, DY, masks, activation)
    got = ref.run_named(_np(params), X.numpy(), DY.numpy(), _np(masks) if masks else None,
                        activation)
    missing = set(want) - set(got)
    assert not missing, missing
    for name, w in want.items():
        np.testing.assert_allclose(got[name], w.numpy(), atol=1e-10, rtol=1e-8, err_msg=name)
        assert ref.CANONICAL.get(name, None) is None or got[name].ndim == len(ref.CANONICAL[name])


def test_masks_change_the_result():
    """A dropped mask term would leave the p>0 run equal to the p=0 run."""
    params, X, DY = tg.make_inputs(2, 6, 2, 8, seed=5, w_std=0.4)
    base = ref.run_named(_np(params), X.numpy(), DY.numpy(), None)
    full = _np(tg.make_masks(2, 6, 2, 8, 0.5, seed=9))
    for site in full:
        got = ref.run_named(_np(params), X.numpy(), DY.numpy(), {site: full[site]})
        assert np.abs(got['SB2'] - base['SB2']).max() > 1e-4, site
        assert np.abs(got['DX'] - base['DX']).max() > 1e-4, site


def test_softmax_against_scipy_and_invariants():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(3, 5, 7, 8)) * 4          # pytorch_module/test_softmax.py:17 sizes
    y = ref.softmax(x, -1)
    np.testing.assert_allclose(y, scipy.special.softmax(x, axis=-1), atol=1e-14)
    np.testing.assert_allclose(y.sum(-1), 1.0, atol=1e-14)
    dy = rng.normal(size=x.shape)
    dx = ref.softmax_backward_data(y, dy, -1)
    np.testing.assert_allclose(dx.sum(-1), 0.0, atol=1e-13)
    xt = torch.from_numpy(x).requires_grad_(True)
    torch.softmax(xt, -1).backward(torch.from_numpy(dy))
    np.testing.assert_allclose(dx, xt.grad.numpy(), atol=1e-13)
    # brute force on one row
    r = x[1, 2, 3]; e = np.exp(r - r.max())
    np.testing.assert_allclose(y[1, 2, 3], e / e.sum(), atol=1e-15)


def test_activations_against_torch():
    x = torch.linspace(-6, 6, 241, dtype=torch.float64).requires_grad_(True)
    dy = torch.cos(torch.arange(241, dtype=torch.float64))
    for name, fn in (('relu', torch.relu), ('gelu', tg.gelu_tanh)):
        x.grad = None
        y = fn(x); y.backward(dy)
        fwd, bwd = ref._ACT[name]
        np.testing.assert_allclose(fwd(x.detach().numpy()), y.detach().numpy(), atol=1e-14)
        np.testing.assert_allclose(bwd(x.detach().numpy(), dy.numpy()), x.grad.numpy(), atol=1e-13)
    # the reference's six-digit constants (transformer.py:25-28) are these
    c = np.sqrt(2 / np.pi)
    for lit, exact in ((0.0356774, 0.044715 * c), (0.797885, c), (0.0535161, 1.5 * 0.044715 * c),
                       (0.398942, 0.5 * c)):
        assert abs(lit - exact) < 1e-6


def test_layer_norm_modes():
    rng = np.random.default_rng(1)
    x = rng.normal(size=(2, 5, 16)) * 3 + 1; s = rng.normal(size=16); b = rng.normal(size=16)
    dy = rng.normal(size=x.shape)
    out, mean, std, normed = ref.layer_norm(x, s, b)
    xt = torch.from_numpy(x).requires_grad_(True)
    st = torch.from_numpy(s).requires_grad_(True); bt = torch.from_numpy(b).requires_grad_(True)
    yt = F.layer_norm(xt, (16,), st, bt, 1e-5); yt.backward(torch.from_numpy(dy))
    np.testing.assert_allclose(out, yt.detach().numpy(), atol=1e-13)
    np.testing.assert_allclose(ref.layer_norm_backward_data(x, dy, mean, std, s), xt.grad.numpy(),
                               atol=1e-12)
    ds, db = ref.layer_norm_backward_weights(dy, normed)
    np.testing.assert_allclose(ds, st.grad.numpy(), atol=1e-12)
    np.testing.assert_allclose(db, bt.grad.numpy(), atol=1e-12)
    # the NumPy reference's eps placement (transformer.py:102) differs by O(eps)
    out2, _, std2, _ = ref.layer_norm(x, s, b, ln_mode='numpy')
    np.testing.assert_allclose(std2, x.std(-1, keepdims=True), atol=0)
    assert 0 < np.abs(out2 - out).max() < 1e-4


def test_fused_op_closed_forms_against_torch():
    """Each op_* closed form against torch functional + autograd."""
    rng = np.random.default_rng(2)
    Bq, J, N, U = 2, 5, 16, 24
    # bdrln / blnrd
    inp = rng.normal(size=(Bq, J, N)); resid = rng.normal(size=(Bq, J, N))
    lb = rng.normal(size=N); s = rng.normal(size=N); b = rng.normal(size=N)
    mask = (rng.random((Bq, J, N)) > 0.3).astype(np.float64)
    lin, istd, diff, normed, out = ref.op_bdrln(inp, resid, lb, s, b, mask)
    it = torch.from_numpy(inp).requires_grad_(True)
    r = (it + torch.from_numpy(lb)) * torch.from_numpy(mask) + torch.from_numpy(resid)
    r.retain_grad()
    o = F.layer_norm(r, (N,), torch.from_numpy(s), torch.from_numpy(b), 1e-5)
    dout = rng.normal(size=out.shape)
    o.backward(torch.from_numpy(dout))
    np.testing.assert_allclose(out, o.detach().numpy(), atol=1e-12)
    np.testing.assert_allclose(lin, inp + lb, atol=0)
    np.testing.assert_allclose(diff, (r - r.mean(-1, keepdim=True)).detach().numpy(), atol=1e-13)
    np.testing.assert_allclose(istd, 1 / np.sqrt(r.detach().numpy().var(-1) + 1e-5), atol=1e-13)
    d_ln_in, d_drop_in = ref.op_blnrd(dout * s, istd, diff, mask)
    np.testing.assert_allclose(d_ln_in, r.grad.numpy(), atol=1e-12)
    np.testing.assert_allclose(d_drop_in, it.grad.numpy(), atol=1e-12)
    # bsb / ebsb
    din, dscale, dbias = ref.op_bsb(normed, s, dout)
    np.testing.assert_allclose(din, dout * s, atol=0)
    np.testing.assert_allclose(dscale, (dout * normed).reshape(-1, N).sum(0), atol=1e-12)
    np.testing.assert_allclose(dbias, dout.reshape(-1, N).sum(0), atol=1e-12)
    d2 = rng.normal(size=dout.shape); dl = rng.normal(size=dout.shape)
    e = ref.op_ebsb(normed, s, dout, d2, dl)
    f3 = ref.op_bsb(normed, s, dout + d2)
    for x, y in zip(e[:3], f3):
        np.testing.assert_allclose(x, y, atol=1e-12)
    np.testing.assert_allclose(e[3], dl.reshape(-1, N).sum(0), atol=1e-12)
    # bad / bdrlb
    for act, fn in (('relu', torch.relu), ('gelu', tg.gelu_tanh)):
        x = rng.normal(size=(Bq, J, U)); bias = rng.normal(size=U)
        m = (rng.random(x.shape) > 0.4).astype(np.float64)
        xt = torch.from_numpy(x).requires_grad_(True); bt = torch.from_numpy(bias).requires_grad_(True)
        y = fn(xt + bt) * torch.from_numpy(m)
        dy = rng.normal(size=x.shape); y.backward(torch.from_numpy(dy))
        lin1, o1 = ref.op_bad(x, bias, m, act)
        np.testing.assert_allclose(o1, y.detach().numpy(), atol=1e-13)
        dlin, dbias1 = ref.op_bdrlb(dy, m, lin1, act)
        np.testing.assert_allclose(dlin, xt.grad.numpy(), atol=1e-12)
        np.testing.assert_allclose(dbias1, bt.grad.numpy(), atol=1e-11)
    # softmax fwd / bs with scaling
    beta = rng.normal(size=(2, 3, 4, 8)); m = (rng.random(beta.shape) > 0.2).astype(np.float64)
    bt = torch.from_numpy(beta).requires_grad_(True)
    y = torch.softmax(bt * 0.125, -1) * torch.from_numpy(m)
    dy = rng.normal(size=beta.shape); y.backward(torch.from_numpy(dy))
    alpha, drop = ref.op_softmax(beta, m, 0.125)
    np.testing.assert_allclose(drop, y.detach().numpy(), atol=1e-14)
    np.testing.assert_allclose(ref.op_bs(alpha, m, dy, 0.125), bt.grad.numpy(), atol=1e-13)
    # aib / baib / baob / bei
    w = rng.normal(size=(3, 4, 2, 2, 5)); bb = rng.normal(size=(3, 4, 2))
    np.testing.assert_allclose(ref.op_aib(w, bb)[1, 2, 1, 0, 3], w[1, 2, 1, 0, 3] + bb[1, 2, 1])
    np.testing.assert_allclose(ref.op_baib(w)[2, 3, 1], w[2, 3, 1].sum(), atol=1e-13)
    np.testing.assert_allclose(ref.op_baob(inp)[5], inp[:, :, 5].sum(), atol=1e-13)
    np.testing.assert_allclose(ref.op_bei(inp, resid), inp + resid)
