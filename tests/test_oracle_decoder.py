"""Pins oracle/decoder_ref.py (substation/transformer.py:288-441) against stock
PyTorch: ``torch.nn.TransformerDecoderLayer`` in fp64, post-norm, no dropout --
forward, dX, the gradient of the encoder output and all 24 parameter gradients.
A dropped residual, a wrong LayerNorm, keys and values taken from the wrong
tensor, a gradient of the encoder output that misses its key or value half, or a
transposed weight each fail one of these comparisons.  The fed-mask dropout paths
are pinned by autograd of the same formula with explicit mask nodes."""
import numpy as np
import pytest
import torch

from oracle import decoder_ref as dref
from oracle import encoder_ref as ref
from tests import torch_graph as tg

B, LT, LS, H, E = 3, 7, 5, 4, 8
P, U = E // H, 4 * E


def _params(seed):
    rng = np.random.default_rng(seed)
    n = lambda *s: rng.normal(size=s) * 0.3
    return dict(
        sattn_wq=n(H, P, E), sattn_wk=n(H, P, E), sattn_wv=n(H, P, E), sattn_wo=n(E, H * P),
        sattn_in_b=n(3, H, P), sattn_out_b=n(E),
        edattn_wq=n(H, P, E), edattn_wk=n(H, P, E), edattn_wv=n(H, P, E), edattn_wo=n(E, H * P),
        edattn_in_b=n(3, H, P), edattn_out_b=n(E),
        norm1_scale=1 + n(E), norm1_bias=n(E), norm2_scale=1 + n(E), norm2_bias=n(E),
        norm3_scale=1 + n(E), norm3_bias=n(E),
        linear1_w=n(U, E), linear1_b=n(U), linear2_w=n(E, U), linear2_b=n(E))


def _run_oracle(p, x, enc, dy, mask, activation, masks=None, relu_gate=None):
    masks = masks or {}
    scale = 1.0 / np.sqrt(P)
    f = dref.decoder_with_encoder_attention(
        x, enc, p['sattn_wq'], p['sattn_wk'], p['sattn_wv'], p['sattn_wo'], p['sattn_in_b'], p['sattn_out_b'],
        scale, mask, p['edattn_wq'], p['edattn_wk'], p['edattn_wv'], p['edattn_wo'], p['edattn_in_b'],
        p['edattn_out_b'], scale, p['norm1_scale'], p['norm1_bias'], p['norm2_scale'], p['norm2_bias'],
        p['norm3_scale'], p['norm3_bias'], p['linear1_w'], p['linear1_b'], p['linear2_w'], p['linear2_b'],
        activation=activation, **masks)
    g = dref.decoder_with_encoder_attention_backward(
        x, enc, dy, f, p['sattn_wq'], p['sattn_wk'], p['sattn_wv'], p['sattn_wo'], scale,
        p['edattn_wq'], p['edattn_wk'], p['edattn_wv'], p['edattn_wo'], scale,
        p['norm1_scale'], p['norm2_scale'], p['norm3_scale'],
        p['linear1_w'], p['linear1_b'], p['linear2_w'], p['linear2_b'], activation=activation,
        relu_gate=relu_gate, **masks)
    return f, g


@pytest.mark.parametrize('activation', ['relu', 'gelu'])
@pytest.mark.parametrize('masked', [False, True])
def test_decoder_matches_torch_transformer_decoder_layer(activation, masked):
    p = _params(3)
    rng = np.random.default_rng(4)
    x, enc, dy = rng.normal(size=(B, LT, E)), rng.normal(size=(B, LS, E)), rng.normal(size=(B, LT, E))
    act = 'relu' if activation == 'relu' else tg.gelu_tanh
    layer = torch.nn.TransformerDecoderLayer(E, H, U, dropout=0.0, activation=act, batch_first=True,
                                             norm_first=False).double()
    T = torch.from_numpy
    with torch.no_grad():
        for mha, pre in ((layer.self_attn, 'sattn'), (layer.multihead_attn, 'edattn')):
            mha.in_proj_weight.copy_(T(np.concatenate([p[pre + '_wq'].reshape(H * P, E),
                                                       p[pre + '_wk'].reshape(H * P, E),
                                                       p[pre + '_wv'].reshape(H * P, E)])))
            mha.in_proj_bias.copy_(T(p[pre + '_in_b'].reshape(-1)))
            mha.out_proj.weight.copy_(T(p[pre + '_wo']))
            mha.out_proj.bias.copy_(T(p[pre + '_out_b']))
        layer.linear1.weight.copy_(T(p['linear1_w'])); layer.linear1.bias.copy_(T(p['linear1_b']))
        layer.linear2.weight.copy_(T(p['linear2_w'])); layer.linear2.bias.copy_(T(p['linear2_b']))
        for i, nm in ((1, layer.norm1), (2, layer.norm2), (3, layer.norm3)):
            nm.weight.copy_(T(p[f'norm{i}_scale'])); nm.bias.copy_(T(p[f'norm{i}_bias']))
    layer.train()
    scale = 1.0 / np.sqrt(P)
    mask = None
    tx, tenc = T(x).requires_grad_(True), T(enc).requires_grad_(True)
    if masked:
        # causal plus finite entries: pins where the mask enters (the raw scores, before
        # the scaling, attention.py:65-68; torch adds its mask after the scaling)
        mask = ref.gen_attn_mask(LT, LT) + np.tril(np.random.default_rng(5).normal(size=(LT, LT)))
        y = layer(tx, tenc, tgt_mask=T(scale * mask))
    else:
        y = layer(tx, tenc)
    y.backward(T(dy))

    f, g = _run_oracle(p, x, enc, dy, mask, activation)
    tol = dict(atol=1e-10, rtol=1e-9)
    np.testing.assert_allclose(f['y'], y.detach().numpy(), **tol)
    np.testing.assert_allclose(g['dx'], tx.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dencoder_out'], tenc.grad.numpy(), **tol)
    for mha, pre in ((layer.self_attn, 'sattn'), (layer.multihead_attn, 'edattn')):
        dw = mha.in_proj_weight.grad.numpy().reshape(3, H, P, E)
        np.testing.assert_allclose(g[f'd{pre}_wq'], dw[0], **tol)
        np.testing.assert_allclose(g[f'd{pre}_wk'], dw[1], **tol)
        np.testing.assert_allclose(g[f'd{pre}_wv'], dw[2], **tol)
        np.testing.assert_allclose(g[f'd{pre}_in_b'], mha.in_proj_bias.grad.numpy().reshape(3, H, P), **tol)
        np.testing.assert_allclose(g[f'd{pre}_wo'], mha.out_proj.weight.grad.numpy(), **tol)
        np.testing.assert_allclose(g[f'd{pre}_out_b'], mha.out_proj.bias.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dlinear1_w'], layer.linear1.weight.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dlinear1_b'], layer.linear1.bias.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dlinear2_w'], layer.linear2.weight.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dlinear2_b'], layer.linear2.bias.grad.numpy(), **tol)
    for i, nm in ((1, layer.norm1), (2, layer.norm2), (3, layer.norm3)):
        np.testing.assert_allclose(g[f'dnorm{i}_scale'], nm.weight.grad.numpy(), **tol)
        np.testing.assert_allclose(g[f'dnorm{i}_bias'], nm.bias.grad.numpy(), **tol)


def _torch_decoder_with_masks(p, x, enc, mask, masks, activation):
    """The layer written with torch operations and explicit {0,1} mask factors at the
    four dropout sites (y = x * mask, no rescale), for autograd."""
    scale = 1.0 / np.sqrt(P)

    def attn(q, kv, pre, m):
        pq = torch.einsum('ble,hpe->bhlp', q, p[pre + '_wq']) + p[pre + '_in_b'][0][None, :, None, :]
        pk = torch.einsum('ble,hpe->bhlp', kv, p[pre + '_wk']) + p[pre + '_in_b'][1][None, :, None, :]
        pv = torch.einsum('ble,hpe->bhlp', kv, p[pre + '_wv']) + p[pre + '_in_b'][2][None, :, None, :]
        s = torch.einsum('bhjp,bhkp->bhjk', pq, pk)
        if m is not None:
            s = s + m
        a = torch.softmax(scale * s, dim=-1)
        w = torch.einsum('bhjk,bhkp->bjhp', a, pv).reshape(q.shape[0], q.shape[1], H * P)
        return w @ p[pre + '_wo'].T + p[pre + '_out_b']

    def ln(t, i):
        mu = t.mean(-1, keepdim=True)
        var = ((t - mu) ** 2).mean(-1, keepdim=True)
        return (t - mu) * torch.rsqrt(var + 1e-5) * p[f'norm{i}_scale'] + p[f'norm{i}_bias']

    act = torch.relu if activation == 'relu' else tg.gelu_tanh
    n1 = ln(attn(x, x, 'sattn', mask) * masks['sattn_dropout_mask'] + x, 1)
    n2 = ln(attn(n1, enc, 'edattn', None) * masks['edattn_dropout_mask'] + n1, 2)
    ff1 = act(n2 @ p['linear1_w'].T + p['linear1_b']) * masks['linear1_dropout_mask']
    return ln((ff1 @ p['linear2_w'].T + p['linear2_b']) * masks['ff_dropout_mask'] + n2, 3)


@pytest.mark.parametrize('activation', ['relu', 'gelu'])
def test_decoder_with_fed_dropout_masks_matches_autograd(activation):
    p = _params(7)
    rng = np.random.default_rng(8)
    x, enc, dy = rng.normal(size=(B, LT, E)), rng.normal(size=(B, LS, E)), rng.normal(size=(B, LT, E))
    masks = dict(sattn_dropout_mask=(rng.random((B, LT, E)) > 0.3).astype(np.float64),
                 edattn_dropout_mask=(rng.random((B, LT, E)) > 0.3).astype(np.float64),
                 linear1_dropout_mask=(rng.random((B, LT, U)) > 0.3).astype(np.float64),
                 ff_dropout_mask=(rng.random((B, LT, E)) > 0.3).astype(np.float64))
    mask = ref.gen_attn_mask(LT, LT)
    T = torch.from_numpy
    tp = {k: T(v).requires_grad_(True) for k, v in p.items()}
    tx, tenc = T(x).requires_grad_(True), T(enc).requires_grad_(True)
    y = _torch_decoder_with_masks(tp, tx, tenc, T(mask), {k: T(v) for k, v in masks.items()}, activation)
    y.backward(T(dy))
    f, g = _run_oracle(p, x, enc, dy, mask, activation, masks)
    tol = dict(atol=1e-10, rtol=1e-9)
    np.testing.assert_allclose(f['y'], y.detach().numpy(), **tol)
    np.testing.assert_allclose(g['dx'], tx.grad.numpy(), **tol)
    np.testing.assert_allclose(g['dencoder_out'], tenc.grad.numpy(), **tol)
    for k in p:
        np.testing.assert_allclose(g['d' + k], tp[k].grad.numpy(), err_msg=k, **tol)
