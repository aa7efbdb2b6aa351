"""CPU oracle of the decoder layer with encoder-decoder attention.  TEST
INFRASTRUCTURE ONLY: imported by tests/ (and nothing that ships).

Restates ``decoder_with_encoder_attention`` and its backward pass,
substation/transformer.py:288-340 and :343-441, on top of the building blocks of
oracle/encoder_ref.py (attention: substation/attention.py:31-179).  As there, the
dropout masks are fed ({0,1}, ``y = x * mask``, no rescale) instead of drawn; the
reference draws none on the attention probabilities of this layer and neither
does this.  LayerNorm uses ``rsqrt(var + eps)`` like the device path
(``ln_mode='numpy'`` gives the script's ``std + eps``).

Pinned by tests/test_oracle_decoder.py against ``torch.nn.TransformerDecoderLayer``
in fp64 (post-norm, forward and every gradient including the one of the encoder
output), which is what the reference's own test/test_transformer_torch.py does for
its layers.
"""
import numpy as np

from .encoder_ref import (_ACT, attn_backward, attn_forward, dropout, dropout_backward_data, layer_norm,
                          layer_norm_backward_data, layer_norm_backward_weights, linear, linear_backward_data,
                          linear_backward_weights)


def decoder_with_encoder_attention(
        x, encoder_out,
        sattn_wq, sattn_wk, sattn_wv, sattn_wo, sattn_in_b, sattn_out_b, sattn_scale, sattn_mask,
        edattn_wq, edattn_wk, edattn_wv, edattn_wo, edattn_in_b, edattn_out_b, edattn_scale,
        norm1_scale, norm1_bias, norm2_scale, norm2_bias, norm3_scale, norm3_bias,
        linear1_w, linear1_b, linear2_w, linear2_b,
        sattn_dropout_mask=None, edattn_dropout_mask=None, linear1_dropout_mask=None, ff_dropout_mask=None,
        activation='gelu', ln_mode='rsqrt'):
    """transformer.py:288-340.  x [B,Lt,E], encoder_out [B,Ls,E]; weights as in
    encoder_ref.attn_forward (wq/wk/wv [H,P,E], wo [E,H*P], in_b [3,H,P] in (q,k,v)
    order); sattn_mask [Lt,Lt] additive or None.  Returns a dict of the output and
    every intermediate the backward pass needs, under the reference's names."""
    act = _ACT[activation][0]
    # masked self-attention, residual, norm1                      transformer.py:299-309
    (sattn, sattn_concat, sattn_proj_q, sattn_proj_k, sattn_proj_v, sattn_alpha, _) = attn_forward(
        x, x, x, sattn_wq, sattn_wk, sattn_wv, sattn_wo, sattn_in_b, sattn_out_b, sattn_scale,
        None, sattn_mask)
    sattn_resid = dropout(sattn, sattn_dropout_mask) + x
    normed1, norm1_mean, norm1_std, norm1_normed = layer_norm(sattn_resid, norm1_scale, norm1_bias, ln_mode=ln_mode)
    # encoder-decoder attention, residual, norm2                  transformer.py:310-321
    (edattn, edattn_concat, edattn_proj_q, edattn_proj_k, edattn_proj_v, edattn_alpha, _) = attn_forward(
        normed1, encoder_out, encoder_out, edattn_wq, edattn_wk, edattn_wv, edattn_wo, edattn_in_b,
        edattn_out_b, edattn_scale)
    edattn_resid = dropout(edattn, edattn_dropout_mask) + normed1
    normed2, norm2_mean, norm2_std, norm2_normed = layer_norm(edattn_resid, norm2_scale, norm2_bias, ln_mode=ln_mode)
    # feed-forward, residual, norm3                               transformer.py:322-331
    ff1_linear = linear(normed2, linear1_w, bias=linear1_b)
    ff1 = dropout(act(ff1_linear), linear1_dropout_mask)
    ff = linear(ff1, linear2_w, bias=linear2_b)
    ff_resid = dropout(ff, ff_dropout_mask) + normed2
    normed3, norm3_mean, norm3_std, norm3_normed = layer_norm(ff_resid, norm3_scale, norm3_bias, ln_mode=ln_mode)
    return dict(y=normed3,
                sattn=sattn, sattn_concat=sattn_concat, sattn_proj_q=sattn_proj_q, sattn_proj_k=sattn_proj_k,
                sattn_proj_v=sattn_proj_v, sattn_scaled_scores=sattn_alpha,
                norm1_mean=norm1_mean, norm1_std=norm1_std, norm1_normed=norm1_normed,
                edattn=edattn, edattn_concat=edattn_concat, edattn_proj_q=edattn_proj_q,
                edattn_proj_k=edattn_proj_k, edattn_proj_v=edattn_proj_v, edattn_scaled_scores=edattn_alpha,
                norm2_mean=norm2_mean, norm2_std=norm2_std, norm2_normed=norm2_normed,
                norm3_mean=norm3_mean, norm3_std=norm3_std, norm3_normed=norm3_normed,
                ff_resid=ff_resid, ff1=ff1, ff1_linear=ff1_linear, normed2=normed2,
                edattn_resid=edattn_resid, normed1=normed1, sattn_resid=sattn_resid)


def decoder_with_encoder_attention_backward(
        x, encoder_out, dy, fwd,
        sattn_wq, sattn_wk, sattn_wv, sattn_wo, sattn_scale,
        edattn_wq, edattn_wk, edattn_wv, edattn_wo, edattn_scale,
        norm1_scale, norm2_scale, norm3_scale,
        linear1_w, linear1_b, linear2_w, linear2_b,
        sattn_dropout_mask=None, edattn_dropout_mask=None, linear1_dropout_mask=None, ff_dropout_mask=None,
        activation='gelu', relu_gate=None):
    """transformer.py:343-441.  ``fwd`` is the forward function's dict.  The masked
    positions of the self-attention have probability zero, so the backward pass
    does not read the mask (attention.py:82-179 never does).  ``relu_gate`` as in
    encoder_ref.encoder_backward.  Returns a dict: dx, dencoder_out and the 24
    parameter gradients under the reference's names (in_b gradients in (q,k,v)
    order)."""
    act_bwd = _ACT[activation][1]
    f = fwd
    # norm3, residual, feed-forward                               transformer.py:371-395
    dff_resid = layer_norm_backward_data(f['ff_resid'], dy, f['norm3_mean'], f['norm3_std'], norm3_scale)
    dnorm3_scale, dnorm3_bias = layer_norm_backward_weights(dy, f['norm3_normed'])
    dff = dropout_backward_data(dff_resid, ff_dropout_mask)
    dff1 = linear_backward_data(f['ff1'], linear2_w, dff)
    dlinear2_w, dlinear2_b = linear_backward_weights(f['ff1'], linear2_w, dff, bias=linear2_b)
    dff1_act = dropout_backward_data(dff1, linear1_dropout_mask)
    if relu_gate is not None and activation == 'relu':
        dff1_linear = relu_gate * dff1_act
    else:
        dff1_linear = act_bwd(f['ff1_linear'], dff1_act)
    dnormed2_linear = linear_backward_data(f['normed2'], linear1_w, dff1_linear)
    dlinear1_w, dlinear1_b = linear_backward_weights(f['normed2'], linear1_w, dff1_linear, bias=linear1_b)
    dnormed2 = dff_resid + dnormed2_linear
    # norm2, residual, encoder-decoder attention                  transformer.py:396-413
    dedattn_resid = layer_norm_backward_data(f['edattn_resid'], dnormed2, f['norm2_mean'], f['norm2_std'], norm2_scale)
    dnorm2_scale, dnorm2_bias = layer_norm_backward_weights(dnormed2, f['norm2_normed'])
    dedattn = dropout_backward_data(dedattn_resid, edattn_dropout_mask)
    (dnormed1_attn, dk, dv, dedattn_wq, dedattn_wk, dedattn_wv, dedattn_wo, dedattn_in_b, dedattn_out_b,
     _, _) = attn_backward(
        f['normed1'], encoder_out, encoder_out, edattn_wq, edattn_wk, edattn_wv, edattn_wo, edattn_scale, dedattn,
        f['edattn_concat'], f['edattn_proj_q'], f['edattn_proj_k'], f['edattn_proj_v'],
        f['edattn_scaled_scores'], f['edattn_scaled_scores'], None, self_attention=False)
    dencoder_out = dk + dv            # keys and values are the same tensor: attention.py:175-177
    dnormed1 = dedattn_resid + dnormed1_attn
    # norm1, residual, self-attention                             transformer.py:414-434
    dsattn_resid = layer_norm_backward_data(f['sattn_resid'], dnormed1, f['norm1_mean'], f['norm1_std'], norm1_scale)
    dnorm1_scale, dnorm1_bias = layer_norm_backward_weights(dnormed1, f['norm1_normed'])
    dsattn = dropout_backward_data(dsattn_resid, sattn_dropout_mask)
    (dx_attn, _, _, dsattn_wq, dsattn_wk, dsattn_wv, dsattn_wo, dsattn_in_b, dsattn_out_b, _, _) = attn_backward(
        x, x, x, sattn_wq, sattn_wk, sattn_wv, sattn_wo, sattn_scale, dsattn,
        f['sattn_concat'], f['sattn_proj_q'], f['sattn_proj_k'], f['sattn_proj_v'],
        f['sattn_scaled_scores'], f['sattn_scaled_scores'], None, self_attention=True)
    dx = dsattn_resid + dx_attn
    return dict(dx=dx, dencoder_out=dencoder_out,
                dsattn_wq=dsattn_wq, dsattn_wk=dsattn_wk, dsattn_wv=dsattn_wv, dsattn_wo=dsattn_wo,
                dsattn_in_b=dsattn_in_b, dsattn_out_b=dsattn_out_b,
                dedattn_wq=dedattn_wq, dedattn_wk=dedattn_wk, dedattn_wv=dedattn_wv, dedattn_wo=dedattn_wo,
                dedattn_in_b=dedattn_in_b, dedattn_out_b=dedattn_out_b,
                dnorm1_scale=dnorm1_scale, dnorm1_bias=dnorm1_bias, dnorm2_scale=dnorm2_scale,
                dnorm2_bias=dnorm2_bias, dnorm3_scale=dnorm3_scale, dnorm3_bias=dnorm3_bias,
                dlinear1_w=dlinear1_w, dlinear1_b=dlinear1_b, dlinear2_w=dlinear2_w, dlinear2_b=dlinear2_b)
