"""The device path's operator graph written with stock torch ops and the einsum
strings of pytorch_module/encoder.cu:87-299, differentiated by torch.autograd.

Independent of oracle/: used to pin the oracle (tests/test_oracle_encoder.py) and
to write the committed fixtures (tests/golden/make_fixtures.py)."""
import math

import torch
import torch.nn.functional as F

PARAM_SHAPES = dict(WKQV='QPHI', BKQV='QPH', WO='IPH', BO='I', S1='I', B1='I', LINB1='U',
                    LINW1='IU', S2='I', B2='I', LINB2='I', LINW2='UI')


def sizes(B, L, H, E, U=None):
    return dict(Q=3, B=B, J=L, K=L, H=H, P=E // H, I=E, U=U or 4 * E)


def make_inputs(B, L, H, E, seed, dtype=torch.float64, w_std=0.02, b_std=0.02, U=None):
    """Synthetic inputs in canonical dim order: X, DY ~ N(0,1); weights N(0,w_std);
    biases N(0,b_std); LN scale 1 + N(0,0.1) and LN bias N(0,0.1) so that their
    gradients are exercised."""
    g = torch.Generator().manual_seed(seed)
    sz = sizes(B, L, H, E, U)
    p = {}
    for name, dims in PARAM_SHAPES.items():
        shape = tuple(sz[d] for d in dims)
        t = torch.randn(shape, generator=g, dtype=torch.float64)
        if name in ('S1', 'S2'):
            t = 1.0 + 0.1 * t
        elif name in ('B1', 'B2'):
            t = 0.1 * t
        elif len(dims) == 1 or name == 'BKQV':
            t = b_std * t
        else:
            t = w_std * t
        p[name] = t.to(dtype)
    X = torch.randn((B, L, E), generator=g, dtype=torch.float64).to(dtype)
    DY = torch.randn((B, L, E), generator=g, dtype=torch.float64).to(dtype)
    return p, X, DY


def make_masks(B, L, H, E, pdrop, seed, dtype=torch.float64, U=None):
    g = torch.Generator().manual_seed(seed + 17)
    sz = sizes(B, L, H, E, U)
    shp = dict(ATTN_DROP_MASK='HBJK', DROP1MASK='BJI', DROP2MASK='BJU', DROP3MASK='BJI')
    return {k: (torch.rand(tuple(sz[d] for d in v), generator=g) >= pdrop).to(dtype)
            for k, v in shp.items()}


def gelu_tanh(x):
    return F.gelu(x, approximate='tanh')


def run(params, X, DY, masks=None, activation='relu', eps=1e-5):
    """Forward + autograd backward.  Returns dict name -> tensor (canonical dims)
    holding every forward intermediate, SB2, DX, 'D'+param, and the backward
    intermediates that are gradients of forward tensors."""
    masks = masks or {}
    p = {k: v.clone().requires_grad_(True) for k, v in params.items()}
    X = X.clone().requires_grad_(True)
    one = lambda name, ref: masks.get(name, torch.ones_like(ref))
    P = p['WKQV'].shape[1]
    t = {}

    def keep(name, v):
        if v.requires_grad:
            v.retain_grad()
        t[name] = v
        return v

    wkk = keep('WKKWQQWVV', torch.einsum('bji,qphi->qphbj', X, p['WKQV']))
    kkqqvv = keep('KKQQVV', wkk + p['BKQV'][..., None, None])
    KK, QQ, VV = kkqqvv[0], kkqqvv[1], kkqqvv[2]
    beta = keep('BETA', torch.einsum('phbk,phbj->hbjk', KK, QQ) / math.sqrt(P))
    alpha = keep('ALPHA', torch.softmax(beta, dim=-1))
    drop = keep('ATTN_DROP', alpha * one('ATTN_DROP_MASK', alpha))
    gamma = keep('GAMMA', torch.einsum('phbk,hbjk->phbj', VV, drop))
    att = keep('ATT', torch.einsum('iph,phbj->bji', p['WO'], gamma) + p['BO'])
    resid1 = att * one('DROP1MASK', att) + X
    keep('RESID1', resid1)
    mu1 = resid1.mean(-1, keepdim=True)
    t['LN1DIFF'] = resid1 - mu1
    t['LN1STD'] = torch.rsqrt(resid1.var(-1, unbiased=False) + eps)
    ln1 = keep('LN1', t['LN1DIFF'] * t['LN1STD'][..., None])
    sb1 = keep('SB1', ln1 * p['S1'] + p['B1'])
    sb1w = keep('SB1_LINW1', torch.einsum('bji,iu->bju', sb1, p['LINW1']))
    lin1 = keep('LIN1', sb1w + p['LINB1'])
    act = torch.relu(lin1) if activation == 'relu' else gelu_tanh(lin1)
    drop2 = keep('DROP2', act * one('DROP2MASK', act))
    d2w = keep('DROP2_LINW2', torch.einsum('bju,ui->bji', drop2, p['LINW2']))
    lin2 = keep('LIN2', d2w + p['LINB2'])
    resid2 = lin2 * one('DROP3MASK', lin2) + sb1
    keep('RESID2', resid2)
    mu2 = resid2.mean(-1, keepdim=True)
    t['LN2DIFF'] = resid2 - mu2
    t['LN2STD'] = torch.rsqrt(resid2.var(-1, unbiased=False) + eps)
    ln2 = keep('LN2', t['LN2DIFF'] * t['LN2STD'][..., None])
    sb2 = keep('SB2', ln2 * p['S2'] + p['B2'])
    sb2.backward(DY)

    out = {k: v.detach() for k, v in t.items()}
    for k, v in p.items():
        out['D' + k] = v.grad.detach()
    out['DX'] = X.grad.detach()
    g = lambda n: t[n].grad.detach()
    out['DLN2'] = g('LN2'); out['DRESID2'] = g('RESID2'); out['DLIN2'] = g('LIN2')
    out['DDROP2'] = g('DROP2'); out['DLIN1'] = g('LIN1')
    out['DLN1'] = g('LN1'); out['DRESID1'] = g('RESID1'); out['DATT'] = g('ATT')
    out['DGAMMA'] = g('GAMMA'); out['DATTN_DROP'] = g('ATTN_DROP'); out['DBETA'] = g('BETA')
    out['DKKQQVV'] = g('KKQQVV')
    # the two partial sums the device path materialises separately
    out['DLIN1_LINW1'] = torch.einsum('bju,iu->bji', out['DLIN1'], params['LINW1'])
    out['DXATT'] = out['DX'] - out['DRESID1']
    del out['RESID1'], out['RESID2']
    return out
