"""Decoder layer with encoder-decoder attention on the MI355X operators.

The reference states this layer in NumPy only (``decoder_with_encoder_attention``
and its backward pass, substation/transformer.py:288-441; its CUDA module covers
the encoder layer alone).  Here it runs on the device as a sequence of the
library's operators -- the contraction kernel with bias and residual addends in
its epilogue, the attention kernels that keep the scores in registers (with an
additive mask for the self-attention and with a key length of their own for the
attention over the encoder output), bdrln / bad and the LayerNorm-backward
operator -- in the order of the reference's statements.

Argument and parameter names follow the reference's (``sattn_*``, ``edattn_*``,
``norm{1,2,3}_*``, ``linear{1,2}_*``).  The three self-attention projections are
one stacked weight, as in the encoder module (index 0 = K, 1 = Q, 2 = V,
pytorch_module/encoder.cu:93-99).  Dropout follows the device contract of the
encoder module: {0,1} masks from the seeded Philox streams, ``y = x * mask``
without rescaling; as in the reference there is none on the attention
probabilities of this layer.
"""
import contextlib
import math

import torch

from .encoder import causal_mask
from .ops import Ops

#: dropout sites (Philox stream ids) of the four masks, in the order of the constructor's probabilities
SITE_SATTN, SITE_EDATTN, SITE_LINEAR1, SITE_FF = 1, 4, 2, 3


class DecoderLayer(torch.nn.Module):
    """``forward(x, encoder_out)``: x [B, target_len, E], encoder_out [B, source_len, E],
    fp16 on the GPU; returns [B, target_len, E].  Sequence lengths must be
    multiples of 128 and the head size 64 or 128 (the attention kernels' tiles)."""

    def __init__(self, batch_size, target_len, source_len, num_heads, embedding_size,
                 sattn_dropout_p=0.1, edattn_dropout_p=0.1, linear1_dropout_p=0.1, ff_dropout_p=0.1,
                 activation='gelu', seed=0, intermediate_size=None, sattn_mask='causal'):
        super().__init__()
        B, Lt, Ls, H, E = batch_size, target_len, source_len, num_heads, embedding_size
        if E % H:
            raise ValueError('embedding_size must be a multiple of num_heads')
        P, U = E // H, intermediate_size or 4 * E
        if Lt % 128 or Ls % 128 or P not in (64, 128):
            raise ValueError('DecoderLayer: sequence lengths must be multiples of 128 and the head size 64 or 128')
        self.batch_size, self.target_len, self.source_len = B, Lt, Ls
        self.num_heads, self.embedding_size, self.proj_size, self.intermediate_size = H, E, P, U
        self.probs = (sattn_dropout_p, edattn_dropout_p, linear1_dropout_p, ff_dropout_p)
        self.activation = activation
        self.seed, self.step = seed, 0
        self.activation_epilogues = True     # linear1 / its backward with the activation in their epilogues where they qualify
        self.ffn_in_epilogues = False        # whether the last forward call took them
        self.ops_t = Ops(B, Lt, H, E, activation=activation, seed=seed, intermediate_size=U)   # target-side sizes
        self.ops_s = Ops(B, Ls, H, E, activation=activation, seed=seed, intermediate_size=U)   # source-side sizes

        def param(*shape, std=None, fill=None):
            t = torch.empty(shape, dtype=torch.float16)
            if fill is not None:
                t.fill_(fill)
            else:
                t.normal_(0.0, std)
            return torch.nn.Parameter(t)

        w = 1.0 / math.sqrt(E)
        self.sattn_wkqv = param(3, H, P, E, std=w)      # [Q,H,P,I], Q: 0 = K, 1 = Q, 2 = V
        self.sattn_in_b = param(3, H, P, fill=0.0)
        self.sattn_wo = param(E, H, P, std=w)
        self.sattn_out_b = param(E, fill=0.0)
        self.edattn_wq = param(H, P, E, std=w)
        self.edattn_wk = param(H, P, E, std=w)
        self.edattn_wv = param(H, P, E, std=w)
        self.edattn_in_b = param(3, H, P, fill=0.0)     # (q, k, v) order, as the reference's in_b
        self.edattn_wo = param(E, H, P, std=w)
        self.edattn_out_b = param(E, fill=0.0)
        for i in (1, 2, 3):
            setattr(self, f'norm{i}_scale', param(E, fill=1.0))
            setattr(self, f'norm{i}_bias', param(E, fill=0.0))
        self.linear1_w = param(U, E, std=w)
        self.linear1_b = param(U, fill=0.0)
        self.linear2_w = param(E, U, std=1.0 / math.sqrt(U))
        self.linear2_b = param(E, fill=0.0)
        self.param_names = [n for n, _ in self.named_parameters()]
        if isinstance(sattn_mask, str):
            if sattn_mask != 'causal':
                raise ValueError("sattn_mask: 'causal', None or an additive [target_len, target_len] tensor")
            sattn_mask = causal_mask(Lt, 'cpu')
        self.register_buffer('sattn_mask', sattn_mask, persistent=False)
        self._function = _make_function(self)

    def set_rng(self, seed, step=0):
        """The four masks of forward call number ``step`` are functions of (seed, step) only."""
        self.seed, self.step = seed, step

    def forward(self, x, encoder_out):
        return self._function.apply(x, encoder_out, *[getattr(self, n) for n in self.param_names])


def _make_function(m):
    o, os_ = m.ops_t, m.ops_s
    names = m.param_names
    scale = 1.0 / math.sqrt(m.proj_size)
    p_sattn, p_edattn, p_linear1, p_ff = m.probs
    Lt, Ls, E = m.target_len, m.source_len, m.embedding_size

    class DecoderFunction(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x, enc, *params):
            if not (x.is_cuda and enc.is_cuda):
                raise RuntimeError('DecoderLayer.forward needs tensors on the GPU')
            w = dict(zip(names, params))
            x, enc = x.contiguous(), enc.contiguous()
            mask = m.sattn_mask
            for ops in (o, os_):
                ops.set_rng(m.seed, m.step)
            m.step += 1
            e = o.empty
            # masked self-attention, residual, norm1                  transformer.py:299-309
            kqv = e('QBJHP')
            o.einsum(x, 'BJI', w['sattn_wkqv'], 'QHPI', kqv, 'QBJHP', addend=w['sattn_in_b'], l_addend='QHP')
            stats1, keep1 = o.attention_workspace(Lt, Lt)
            gamma1 = e('BJHP')
            o.attention_forward(kqv[1], 'BJHP', kqv[0], kqv[2], 'BKHP', gamma1, 'BJHP', stats1, keep1, scale,
                                attn_mask=mask)
            att1 = e('BJI')
            o.einsum(w['sattn_wo'], 'IHP', gamma1, 'BJHP', att1, 'BJI')
            mask1, diff1, ln1, normed1, istd1 = e('BJI'), e('BJI'), e('BJI'), e('BJI'), e('BJ')
            o.bdrln(att1, 'BJI', x, 'BJI', w['sattn_out_b'], w['norm1_scale'], w['norm1_bias'], att1, 'BJI',
                    mask1, 'BJI', diff1, 'BJI', ln1, 'BJI', normed1, 'BJI', istd1, 'BJ', p=p_sattn, site=SITE_SATTN)
            # encoder-decoder attention, residual, norm2              transformer.py:310-321
            q2, k2, v2 = e('BJHP'), os_.empty('BKHP'), os_.empty('BKHP')
            o.einsum(normed1, 'BJI', w['edattn_wq'], 'HPI', q2, 'BJHP', addend=w['edattn_in_b'][0], l_addend='HP')
            os_.einsum(enc, 'BKI', w['edattn_wk'], 'HPI', k2, 'BKHP', addend=w['edattn_in_b'][1], l_addend='HP')
            os_.einsum(enc, 'BKI', w['edattn_wv'], 'HPI', v2, 'BKHP', addend=w['edattn_in_b'][2], l_addend='HP')
            stats2, keep2 = o.attention_workspace(Lt, Ls)
            gamma2 = e('BJHP')
            o.attention_forward(q2, 'BJHP', k2, v2, 'BKHP', gamma2, 'BJHP', stats2, keep2, scale)
            att2 = e('BJI')
            o.einsum(w['edattn_wo'], 'IHP', gamma2, 'BJHP', att2, 'BJI')
            mask2, diff2, ln2, normed2, istd2 = e('BJI'), e('BJI'), e('BJI'), e('BJI'), e('BJ')
            o.bdrln(att2, 'BJI', normed1, 'BJI', w['edattn_out_b'], w['norm2_scale'], w['norm2_bias'], att2, 'BJI',
                    mask2, 'BJI', diff2, 'BJI', ln2, 'BJI', normed2, 'BJI', istd2, 'BJ', p=p_edattn,
                    site=SITE_EDATTN)
            # feed-forward, residual, norm3                           transformer.py:322-331
            # linear1 with bias, activation and dropout in its epilogue where the product qualifies (the keep bits
            # then travel as bits, no mask tensor; ReLU needs no pre-activation either); else operator by operator
            ff1 = e('BJU')
            lin1 = e('BJU') if m.activation != 'relu' else None
            bits = torch.empty(ff1.numel() // 8, dtype=torch.uint8, device=ff1.device)
            mask3 = None
            if not (m.activation_epilogues and
                    o.einsum_bad(normed2, 'BJI', w['linear1_w'], 'UI', w['linear1_b'], 'U', lin1, ff1, 'BJU', bits,
                                 p=p_linear1, site=SITE_LINEAR1)):
                bits = None
                lin1, mask3 = e('BJU'), e('BJU')
                o.einsum(normed2, 'BJI', w['linear1_w'], 'UI', lin1, 'BJU')
                o.bad(lin1, 'BJU', w['linear1_b'], lin1, 'BJU', mask3, 'BJU', ff1, 'BJU', p=p_linear1,
                      site=SITE_LINEAR1)
            m.ffn_in_epilogues = bits is not None
            ff = e('BJI')
            o.einsum(ff1, 'BJU', w['linear2_w'], 'IU', ff, 'BJI')
            mask4, diff3, ln3, y, istd3 = e('BJI'), e('BJI'), e('BJI'), e('BJI'), e('BJ')
            o.bdrln(ff, 'BJI', normed2, 'BJI', w['linear2_b'], w['norm3_scale'], w['norm3_bias'], ff, 'BJI',
                    mask4, 'BJI', diff3, 'BJI', ln3, 'BJI', y, 'BJI', istd3, 'BJ', p=p_ff, site=SITE_FF)
            ctx.save_for_backward(x, enc, *params)
            ctx.saved = dict(kqv=kqv, stats1=stats1, keep1=keep1, gamma1=gamma1, mask1=mask1, diff1=diff1, ln1=ln1,
                             normed1=normed1, istd1=istd1, q2=q2, k2=k2, v2=v2, stats2=stats2, keep2=keep2,
                             gamma2=gamma2, mask2=mask2, diff2=diff2, ln2=ln2, normed2=normed2, istd2=istd2,
                             lin1=lin1, mask3=mask3, ff1=ff1, bits=bits, mask4=mask4, diff3=diff3, ln3=ln3, istd3=istd3,
                             mask=mask)
            m.last_masks = dict(sattn=mask1, edattn=mask2, linear1=mask3, ff=mask4)
            return y

        @staticmethod
        def backward(ctx, dy):
            x, enc, *params = ctx.saved_tensors
            w = dict(zip(names, params))
            s = ctx.saved
            dy = dy.contiguous()
            # the second stage of every column sum of the pass (eight bias / scale gradients) in one launch at its end
            with contextlib.ExitStack() as stack:
                for ops in ({id(o): o, id(os_): os_}).values():
                    stack.enter_context(ops.deferred_column_sums())
                return DecoderFunction._backward(w, s, x, enc, dy)

        @staticmethod
        def _backward(w, s, x, enc, dy):
            e = o.empty
            g = {n: torch.empty_like(w[n]) for n in names}
            # norm3, residual, feed-forward                           transformer.py:371-395
            dln3, dres3, dff = e('BJI'), e('BJI'), e('BJI')
            o.ln_backward(s['ln3'], 'BJI', w['norm3_scale'], dy, 'BJI', s['istd3'], 'BJ', s['diff3'], 'BJI',
                          s['mask4'], 'BJI', dln3, 'BJI', dres3, 'BJI', dff, 'BJI', g['norm3_scale'], g['norm3_bias'])
            dlin1 = e('BJU')
            gate = s['ff1'] if m.activation == 'relu' else s['lin1']
            if s['bits'] is None or not o.einsum_bdrlb(dff, 'BJI', w['linear2_w'], 'IU', gate, 'BJU', s['bits'],
                                                       dlin1, 'BJU', g['linear1_b']):
                if s['mask3'] is None:
                    raise RuntimeError('DecoderLayer: the forward pass ran linear1 with its activation epilogue, the '
                                       'backward pass cannot (tensors not 16-byte aligned?)')
                dff1 = e('BJU')
                o.einsum(dff, 'BJI', w['linear2_w'], 'IU', dff1, 'BJU')
                o.bdrlb(dff1, 'BJU', s['mask3'], 'BJU', s['lin1'], 'BJU', dlin1, 'BJU', g['linear1_b'])
            o.einsum(dff, 'BJI', s['ff1'], 'BJU', g['linear2_w'], 'IU')
            dnormed2_linear = e('BJI')
            o.einsum_pair((dlin1, 'BJU', w['linear1_w'], 'UI', dnormed2_linear, 'BJI'),
                          (dlin1, 'BJU', s['normed2'], 'BJI', g['linear1_w'], 'UI'))
            # norm2, residual, encoder-decoder attention              transformer.py:396-413
            dln2, dres2, datt2 = e('BJI'), e('BJI'), e('BJI')
            o.ln_backward(s['ln2'], 'BJI', w['norm2_scale'], dres3, 'BJI', s['istd2'], 'BJ', s['diff2'], 'BJI',
                          s['mask2'], 'BJI', dln2, 'BJI', dres2, 'BJI', datt2, 'BJI', g['norm2_scale'], g['norm2_bias'],
                          dout2=dnormed2_linear, l_dout2='BJI', dlinear=dff, l_dlinear='BJI',
                          dlinear_bias=g['linear2_b'], dout_bias=g['edattn_out_b'])
            dgamma2 = e('BJHP')
            o.einsum_pair((w['edattn_wo'], 'IHP', datt2, 'BJI', dgamma2, 'BJHP'),
                          (datt2, 'BJI', s['gamma2'], 'BJHP', g['edattn_wo'], 'IHP'))
            dq2, dk2, dv2 = e('BJHP'), os_.empty('BKHP'), os_.empty('BKHP')
            o.attention_backward(s['q2'], 'BJHP', s['k2'], s['v2'], 'BKHP', s['gamma2'], 'BJHP', dgamma2, 'BJHP',
                                 s['stats2'], s['keep2'], dq2, 'BJHP', dk2, dv2, 'BKHP', scale,
                                 dq_bias=g['edattn_in_b'][0], dk_bias=g['edattn_in_b'][1], dv_bias=g['edattn_in_b'][2])
            dnormed1_attn = e('BJI')
            o.einsum_pair((dq2, 'BJHP', w['edattn_wq'], 'HPI', dnormed1_attn, 'BJI'),
                          (dq2, 'BJHP', s['normed1'], 'BJI', g['edattn_wq'], 'HPI'))
            denc = os_.empty('BKI')
            os_.einsum_pair((dk2, 'BKHP', w['edattn_wk'], 'HPI', denc, 'BKI'),
                            (dk2, 'BKHP', enc, 'BKI', g['edattn_wk'], 'HPI'))
            os_.einsum_pair((dv2, 'BKHP', w['edattn_wv'], 'HPI', denc, 'BKI', denc, 'BKI'),
                            (dv2, 'BKHP', enc, 'BKI', g['edattn_wv'], 'HPI'))
            # norm1, residual, self-attention                         transformer.py:414-434
            dln1, dres1, datt1 = e('BJI'), e('BJI'), e('BJI')
            unused = torch.empty_like(g['sattn_out_b'])          # the column sums of the third input are not needed here
            o.ln_backward(s['ln1'], 'BJI', w['norm1_scale'], dres2, 'BJI', s['istd1'], 'BJ', s['diff1'], 'BJI',
                          s['mask1'], 'BJI', dln1, 'BJI', dres1, 'BJI', datt1, 'BJI', g['norm1_scale'], g['norm1_bias'],
                          dout2=dnormed1_attn, l_dout2='BJI', dlinear=datt2, l_dlinear='BJI',
                          dlinear_bias=unused, dout_bias=g['sattn_out_b'])
            dgamma1 = e('BJHP')
            o.einsum_pair((w['sattn_wo'], 'IHP', datt1, 'BJI', dgamma1, 'BJHP'),
                          (datt1, 'BJI', s['gamma1'], 'BJHP', g['sattn_wo'], 'IHP'))
            dkqv = e('QBJHP')
            kqv = s['kqv']
            o.attention_backward(kqv[1], 'BJHP', kqv[0], kqv[2], 'BKHP', s['gamma1'], 'BJHP', dgamma1, 'BJHP',
                                 s['stats1'], s['keep1'], dkqv[1], 'BJHP', dkqv[0], dkqv[2], 'BKHP', scale,
                                 attn_mask=s['mask'], dq_bias=g['sattn_in_b'][1], dk_bias=g['sattn_in_b'][0],
                                 dv_bias=g['sattn_in_b'][2])
            dx = e('BJI')
            o.einsum_pair((w['sattn_wkqv'], 'QHPI', dkqv, 'QBJHP', dx, 'BJI', dres1, 'BJI'),
                          (dkqv, 'QBJHP', x, 'BJI', g['sattn_wkqv'], 'QHPI'))
            return (dx, denc) + tuple(g[n] for n in names)

    return DecoderFunction
