"""Parity of the decoder layer with encoder-decoder attention
(substation_amd.DecoderLayer, the device counterpart of
substation/transformer.py:288-441) against oracle/decoder_ref.py: output, dX, the
gradient of the encoder output and all parameter gradients within 1e-2 relative
(helpers.assert_close), the four dropout masks exactly equal to the seeded oracle
masks and fed to the oracle.  GELU: with ReLU a pre-activation that fp16 rounds to
the other side of zero flips whole gradient elements, which says nothing about
the layer."""
import numpy as np
import pytest
import torch

from oracle import decoder_ref as dref
from oracle import philox_ref as ph
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu
SEED = 0x5EED + 9


def _f64(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def _oracle_params(layer):
    H, P, E = layer.num_heads, layer.proj_size, layer.embedding_size
    w = {n: _f64(getattr(layer, n)) for n in layer.param_names}
    p = dict(sattn_wq=w['sattn_wkqv'][1], sattn_wk=w['sattn_wkqv'][0], sattn_wv=w['sattn_wkqv'][2],
             sattn_wo=w['sattn_wo'].reshape(E, H * P), sattn_in_b=w['sattn_in_b'][[1, 0, 2]],
             sattn_out_b=w['sattn_out_b'],
             edattn_wq=w['edattn_wq'], edattn_wk=w['edattn_wk'], edattn_wv=w['edattn_wv'],
             edattn_wo=w['edattn_wo'].reshape(E, H * P), edattn_in_b=w['edattn_in_b'],
             edattn_out_b=w['edattn_out_b'])
    for k in ('norm1_scale', 'norm1_bias', 'norm2_scale', 'norm2_bias', 'norm3_scale', 'norm3_bias',
              'linear1_w', 'linear1_b', 'linear2_w', 'linear2_b'):
        p[k] = w[k]
    return p


@pytest.mark.parametrize('dims,p,masked', [
    ((2, 128, 256, 2, 128), 0.1, True),        # target shorter than source, head size 64, causal self-attention
    ((2, 256, 128, 2, 256), 0.0, True),        # target longer than source, head size 128
    ((3, 128, 128, 4, 256), 0.2, False),       # no mask on the self-attention
    ((8, 512, 256, 4, 256, 4096), 0.1, True),  # 16 x 16 tiles of 256 x 256 in the feed-forward products: linear1 and
                                               # its backward carry the activation in their epilogues
])
def test_decoder_layer_matches_the_oracle(dims, p, masked):
    from substation_amd import DecoderLayer
    from substation_amd.decoder import SITE_EDATTN, SITE_FF, SITE_LINEAR1, SITE_SATTN
    B, Lt, Ls, H, E = dims[:5]
    torch.manual_seed(Lt + Ls + H)
    layer = DecoderLayer(B, Lt, Ls, H, E, p, p, p, p, activation='gelu', seed=SEED,
                         sattn_mask='causal' if masked else None,
                         intermediate_size=dims[5] if len(dims) > 5 else None).cuda()
    with torch.no_grad():      # biases and norms away from their trivial initial values
        for n in layer.param_names:
            q = getattr(layer, n)
            if q.dim() == 1 or n.endswith('in_b'):
                q.add_(0.1 * torch.randn_like(q))
    g = torch.Generator().manual_seed(5)
    x = torch.randn(B, Lt, E, generator=g).half().cuda().requires_grad_(True)
    enc = torch.randn(B, Ls, E, generator=g).half().cuda().requires_grad_(True)
    dy = torch.randn(B, Lt, E, generator=g).half().cuda()
    layer.set_rng(SEED, 3)
    y = layer(x, enc)
    y.backward(dy)
    torch.cuda.synchronize()

    U = layer.intermediate_size
    want_masks = dict(sattn=ph.dropout_mask((B, Lt, E), p, SEED, SITE_SATTN, step=3, dtype=np.float64),
                      edattn=ph.dropout_mask((B, Lt, E), p, SEED, SITE_EDATTN, step=3, dtype=np.float64),
                      linear1=ph.dropout_mask((B, Lt, U), p, SEED, SITE_LINEAR1, step=3, dtype=np.float64),
                      ff=ph.dropout_mask((B, Lt, E), p, SEED, SITE_FF, step=3, dtype=np.float64))
    assert layer.ffn_in_epilogues == (len(dims) > 5)
    for k, v in want_masks.items():
        if k == 'linear1' and layer.ffn_in_epilogues:
            continue        # no mask tensor on that path: a wrong keep bit shows in y and in every gradient below
        assert (_f64(layer.last_masks[k]) == v).all(), k + ' mask differs from the seeded oracle mask'

    op = _oracle_params(layer)
    scale = 1.0 / np.sqrt(layer.proj_size)
    mask = _f64(layer.sattn_mask) if masked else None
    f = dref.decoder_with_encoder_attention(
        _f64(x), _f64(enc), op['sattn_wq'], op['sattn_wk'], op['sattn_wv'], op['sattn_wo'], op['sattn_in_b'],
        op['sattn_out_b'], scale, mask, op['edattn_wq'], op['edattn_wk'], op['edattn_wv'], op['edattn_wo'],
        op['edattn_in_b'], op['edattn_out_b'], scale, op['norm1_scale'], op['norm1_bias'], op['norm2_scale'],
        op['norm2_bias'], op['norm3_scale'], op['norm3_bias'], op['linear1_w'], op['linear1_b'], op['linear2_w'],
        op['linear2_b'], sattn_dropout_mask=want_masks['sattn'], edattn_dropout_mask=want_masks['edattn'],
        linear1_dropout_mask=want_masks['linear1'], ff_dropout_mask=want_masks['ff'], activation='gelu')
    gr = dref.decoder_with_encoder_attention_backward(
        _f64(x), _f64(enc), _f64(dy), f, op['sattn_wq'], op['sattn_wk'], op['sattn_wv'], op['sattn_wo'], scale,
        op['edattn_wq'], op['edattn_wk'], op['edattn_wv'], op['edattn_wo'], scale, op['norm1_scale'],
        op['norm2_scale'], op['norm3_scale'], op['linear1_w'], op['linear1_b'], op['linear2_w'], op['linear2_b'],
        sattn_dropout_mask=want_masks['sattn'], edattn_dropout_mask=want_masks['edattn'],
        linear1_dropout_mask=want_masks['linear1'], ff_dropout_mask=want_masks['ff'], activation='gelu')

    H, P = layer.num_heads, layer.proj_size
    assert_close(_f64(y), f['y'], name='y')
    assert_close(_f64(x.grad), gr['dx'], name='dx')
    assert_close(_f64(enc.grad), gr['dencoder_out'], name='dencoder_out')
    got = {n: _f64(getattr(layer, n).grad) for n in layer.param_names}
    assert_close(got['sattn_wkqv'][1], gr['dsattn_wq'], name='dsattn_wq')
    assert_close(got['sattn_wkqv'][0], gr['dsattn_wk'], name='dsattn_wk')
    assert_close(got['sattn_wkqv'][2], gr['dsattn_wv'], name='dsattn_wv')
    assert_close(got['sattn_in_b'][[1, 0, 2]], gr['dsattn_in_b'], name='dsattn_in_b')
    assert_close(got['sattn_wo'].reshape(E, H * P), gr['dsattn_wo'], name='dsattn_wo')
    assert_close(got['edattn_wo'].reshape(E, H * P), gr['dedattn_wo'], name='dedattn_wo')
    for n in ('sattn_out_b', 'edattn_wq', 'edattn_wk', 'edattn_wv', 'edattn_in_b', 'edattn_out_b', 'norm1_scale',
              'norm1_bias', 'norm2_scale', 'norm2_bias', 'norm3_scale', 'norm3_bias', 'linear1_w', 'linear1_b',
              'linear2_w', 'linear2_b'):
        assert_close(got[n], gr['d' + n], name='d' + n)


def test_decoder_layer_steps_draw_new_masks_and_rejects_unsupported_sizes():
    from substation_amd import DecoderLayer
    layer = DecoderLayer(1, 128, 128, 2, 128, 0.5, 0.5, 0.5, 0.5, seed=SEED).cuda()
    x = torch.randn(1, 128, 128).half().cuda()
    enc = torch.randn(1, 128, 128).half().cuda()
    with torch.no_grad():
        layer.set_rng(SEED, 0)
        a = layer(x, enc).clone(); m0 = layer.last_masks['ff'].clone()
        b = layer(x, enc).clone(); m1 = layer.last_masks['ff'].clone()
        layer.set_rng(SEED, 0)
        c = layer(x, enc).clone()
    assert not torch.equal(m0, m1) and not torch.equal(a, b)
    assert torch.equal(a, c)
    with pytest.raises(ValueError):
        DecoderLayer(1, 100, 128, 2, 128)          # target length not a multiple of 128
    with pytest.raises(ValueError):
        DecoderLayer(1, 128, 128, 4, 128)          # head size 32


@pytest.mark.parametrize('activation', ['relu', 'gelu'])
def test_decoder_activation_epilogues_match_the_operators(activation):
    """linear1 with bias, activation and dropout in its epilogue and the backward of that in
    the epilogue of the product before it (sub_op_einsum_bad, sub_op_einsum_bdrlb) against
    the same layer run operator by operator: output and every gradient bit for bit, the
    bias gradient of linear1 (column sums added in another order) to rounding."""
    from substation_amd import DecoderLayer
    B, Lt, Ls, H, E, U = 8, 512, 128, 4, 256, 4096
    outs = []
    for fused in (True, False):
        torch.manual_seed(1)
        layer = DecoderLayer(B, Lt, Ls, H, E, 0.1, 0.1, 0.1, 0.1, activation=activation, seed=SEED,
                             intermediate_size=U).cuda()
        layer.activation_epilogues = fused
        g = torch.Generator().manual_seed(5)
        x = torch.randn(B, Lt, E, generator=g).half().cuda().requires_grad_(True)
        enc = torch.randn(B, Ls, E, generator=g).half().cuda().requires_grad_(True)
        dy = torch.randn(B, Lt, E, generator=g).half().cuda()
        layer.set_rng(SEED, 1)
        y = layer(x, enc)
        y.backward(dy)
        torch.cuda.synchronize()
        assert layer.ffn_in_epilogues == fused
        outs.append([('y', y.detach().clone()), ('dx', x.grad.clone()), ('denc', enc.grad.clone())] +
                    [('d' + n, getattr(layer, n).grad.clone()) for n in layer.param_names])
    for (name, a), (_, b) in zip(*outs):
        assert torch.isfinite(a.float()).all() and float(a.float().abs().max()) > 0, name
        if name == 'dlinear1_b':
            assert_close(_f64(a), _f64(b), tol=2e-3, name=name)
        else:
            assert torch.equal(a, b), name
