"""NumPy restatement of the reference's encoder-layer math.  TEST INFRASTRUCTURE ONLY.

This file is the checker for the HIP path (and the timed CPU baseline); the
product never imports it.  Each function cites the reference lines it follows
(paths relative to the reference checkout).

Differences from ``substation/transformer.py`` that are deliberate, because the
drop-in target is the CUDA module (``pytorch_module/encoder.cu``), not the NumPy
script:

* dropout takes the mask as an INPUT, mask values are {0,1} and kept elements
  are not rescaled (``pytorch_module/blocks.cuh:24-45``); the NumPy reference
  draws ``np.random.choice([0, 1/p])`` internally (``transformer.py:134-138``);
* there is a fourth dropout site on the softmax output
  (``pytorch_module/encoder.cu:120``) that the NumPy encoder lacks;
* layer norm defaults to ``(x-mean)*rsqrt(var+eps)`` and reports the INVERSE
  standard deviation (``pytorch_module/block_bdrln.cuh:254-260``); pass
  ``ln_mode='numpy'`` for ``(x-mean)/(std+eps)`` (``transformer.py:100-102``).

How every function here is pinned (tests/test_oracle_*.py): forward, dX and all
parameter gradients against ``torch.nn.TransformerEncoderLayer`` /
``torch.nn.MultiheadAttention`` / ``torch.nn.functional`` with the weight mapping
of ``test/test_transformer_torch.py:129-141,231-296``; the four dropout sites
against torch autograd of the same graph with explicit ``* mask`` nodes; softmax
against ``scipy.special.softmax`` and its invariants; the committed fixtures in
``tests/golden/``.  No function is left "parity unpinned".
"""

import numpy as np


# --------------------------------------------------------------------------
# activations                                   substation/transformer.py:11-38
# --------------------------------------------------------------------------

_SQRT_2_OVER_PI = np.sqrt(2.0 / np.pi)


def gelu(x):
    """tanh-form GELU, transformer.py:11-14."""
    return 0.5 * x * (1 + np.tanh(_SQRT_2_OVER_PI * (x + 0.044715 * (x ** 3))))


def gelu_backward_data(x, dy):
    """d gelu / dx * dy, transformer.py:17-28.

    The reference hard-codes 0.0356774, 0.797885, 0.0535161, 0.398942; they are
    0.044715*sqrt(2/pi), sqrt(2/pi), 1.5*0.044715*sqrt(2/pi), 0.5*sqrt(2/pi)
    rounded to six digits.  The exact constants are used here.
    """
    c = _SQRT_2_OVER_PI
    inner = c * (x + 0.044715 * x ** 3)
    t = np.tanh(inner)
    sech2 = 1.0 - t * t
    return (0.5 * t + (1.5 * 0.044715 * c * x ** 3 + 0.5 * c * x) * sech2 + 0.5) * dy


def relu(x):
    """transformer.py:31-33."""
    return np.maximum(0, x)


def relu_backward_data(x, dy):
    """transformer.py:36-38."""
    return (x > 0) * dy


_ACT = {'relu': (relu, relu_backward_data), 'gelu': (gelu, gelu_backward_data)}


# --------------------------------------------------------------------------
# linear                                        substation/transformer.py:41-83
# --------------------------------------------------------------------------

def linear(x, w, bias=None):
    """x[..., in] @ w[out, in].T (+ bias), transformer.py:41-52."""
    y = np.matmul(x, w.T)
    return y + bias if bias is not None else y


def linear_backward_data(x, w, dy):
    """transformer.py:55-63."""
    return np.matmul(dy, w)


def linear_backward_weights(x, w, dy, bias=None):
    """(dw[out,in], dbias[out]); 3-d x only, transformer.py:66-83."""
    dbias = dy.sum(axis=(1, 0)) if bias is not None else None
    dw = np.matmul(np.swapaxes(dy, -1, -2), x).sum(axis=0)
    return dw, dbias


# --------------------------------------------------------------------------
# layer norm                                    substation/transformer.py:86-131
# --------------------------------------------------------------------------

def layer_norm(x, scale, bias, eps=1e-5, ln_mode='rsqrt'):
    """Returns (out, mean, std_eff, normed) over the last axis.

    ``std_eff`` is the number the normalisation divides by: ``sqrt(var+eps)`` in
    'rsqrt' mode (block_bdrln.cuh:81-91; the device tensor LN*STD holds its
    inverse), ``std`` itself in 'numpy' mode where the division is by
    ``std+eps`` (transformer.py:100-102) but backward uses ``std`` (:115-117).
    Variance is the biased one (1/n), as in both references.
    """
    mean = x.mean(axis=-1, keepdims=True)
    if ln_mode == 'rsqrt':
        std_eff = np.sqrt(x.var(axis=-1, keepdims=True) + eps)
        normed = (x - mean) / std_eff
    elif ln_mode == 'numpy':
        std_eff = x.std(axis=-1, keepdims=True)
        normed = (x - mean) / (std_eff + eps)
    else:
        raise ValueError('ln_mode must be "rsqrt" or "numpy"')
    return normed * scale + bias, mean, std_eff, normed


def layer_norm_backward_data(x, dy, mean, std, scale=None):
    """transformer.py:108-118."""
    n = x.shape[-1]
    scaled_dy = dy * scale if scale is not None else dy
    dmean = -scaled_dy.sum(axis=-1, keepdims=True) / std
    dstd = -(scaled_dy * (x - mean)).sum(axis=-1, keepdims=True) / (std ** 2)
    return scaled_dy / std + dmean / n + dstd * (x - mean) / n / std


def layer_norm_backward_weights(dy, normed):
    """(dscale, dbias), transformer.py:121-131."""
    return (normed * dy).sum(axis=1).sum(axis=0), dy.sum(axis=1).sum(axis=0)


# --------------------------------------------------------------------------
# dropout with a fed mask     transformer.py:134-148, pytorch_module/blocks.cuh:44
# --------------------------------------------------------------------------

def dropout(x, mask):
    """y = x*mask; ``mask is None`` means p = 0 (transformer.py:136)."""
    return x if mask is None else x * mask


def dropout_backward_data(dy, mask):
    """transformer.py:141-148."""
    return dy if mask is None else dy * mask


# --------------------------------------------------------------------------
# softmax                                        substation/attention.py:14-28
# --------------------------------------------------------------------------

def softmax(x, dim=-1):
    """attention.py:14-17."""
    exps = np.exp(x - x.max(axis=dim, keepdims=True))
    return exps / exps.sum(axis=dim, keepdims=True)


def softmax_backward_data(y, dy, dim=-1):
    """attention.py:20-28 (takes the softmax OUTPUT y)."""
    elem_prod = y * dy
    return elem_prod - y * elem_prod.sum(axis=dim, keepdims=True)


# --------------------------------------------------------------------------
# multi-head attention                           substation/attention.py:31-179
# --------------------------------------------------------------------------

def gen_attn_mask(lq, lk, dtype=np.float64):
    """Causal additive mask, transformer.py:151-157: -inf above the diagonal."""
    return np.triu(np.full((lq, lk), float('-inf'), dtype=dtype), k=1)


def attn_forward(q, k, v, wq, wk, wv, wo, in_b, out_b, scale, softmax_mask=None, attn_mask=None):
    """attention.py:31-79, plus the softmax-output dropout of encoder.cu:120.

    q,k,v [B,L,E]; wq,wk,wv [H,P,E]; wo [E,H*P]; in_b [3,H,P] in (q,k,v) order;
    softmax_mask [B,H,Lq,Lk] of {0,1} or None (dropout of the softmax output);
    attn_mask [Lq,Lk] additive or None, added to the raw scores BEFORE the
    scaling as at attention.py:65-68 (a 0/-inf mask is indifferent to that).  Same per-sample loop of
    ``np.matmul`` over the head axis as the reference.  Returns
    (out [B,Lq,E], concat, proj_q, proj_k, proj_v, alpha, attn_drop) with the
    five/six intermediates as per-sample lists like the reference's.
    """
    out = np.empty((q.shape[0], q.shape[-2], wo.shape[0]), dtype=q.dtype)
    proj_q_, proj_k_, proj_v_, concat_, alpha_, drop_ = [], [], [], [], [], []
    for b in range(q.shape[0]):
        proj_q = np.matmul(q[b], wq.transpose(0, 2, 1)) + np.expand_dims(in_b[0], axis=1)
        proj_k = np.matmul(k[b], wk.transpose(0, 2, 1)) + np.expand_dims(in_b[1], axis=1)
        proj_v = np.matmul(v[b], wv.transpose(0, 2, 1)) + np.expand_dims(in_b[2], axis=1)
        scores = np.matmul(proj_q, proj_k.transpose(0, 2, 1))       # [H,Lq,Lk]
        if attn_mask is not None:
            scores = scores + attn_mask
        alpha = softmax(scale * scores, dim=-1)
        attn_drop = dropout(alpha, None if softmax_mask is None else softmax_mask[b])
        weighted = np.matmul(attn_drop, proj_v)                      # [H,Lq,P]
        concat = weighted.transpose(1, 0, 2).reshape(
            weighted.shape[1], weighted.shape[0] * weighted.shape[2])
        out[b] = np.matmul(concat, wo.T) + out_b
        proj_q_.append(proj_q); proj_k_.append(proj_k); proj_v_.append(proj_v)
        concat_.append(concat); alpha_.append(alpha); drop_.append(attn_drop)
    return out, concat_, proj_q_, proj_k_, proj_v_, alpha_, drop_


def attn_backward(q, k, v, wq, wk, wv, wo, scale, dy, concat, proj_q, proj_k, proj_v,
                  alpha, attn_drop, softmax_mask=None, self_attention=True):
    """attention.py:82-179 with the softmax dropout threaded through.

    Returns (dq, dk, dv, dwq, dwk, dwv, dwo, din_b[3,H,P] (q,k,v order), dout_b,
    dalpha_list, dscaled_list) where the last two are per-sample [H,Lq,Lk]
    gradients w.r.t. the dropped softmax output and w.r.t. the SCALED scores
    (the device tensors DATTN_DROP and DBETA).  With ``self_attention`` the
    three input gradients are summed into each other as at attention.py:167-178.
    """
    dq = np.zeros_like(q); dk = np.zeros_like(k); dv = np.zeros_like(v)
    dwq = np.zeros_like(wq); dwk = np.zeros_like(wk); dwv = np.zeros_like(wv)
    dwo = np.zeros_like(wo)
    din_b = np.zeros((3, wq.shape[0], wq.shape[1]), dtype=q.dtype)
    dout_b = np.zeros(wo.shape[0], dtype=q.dtype)
    ddrop_, dbeta_ = [], []
    H, P = wq.shape[0], wq.shape[1]
    for b in range(q.shape[0]):
        dconcat = np.matmul(dy[b], wo)
        dwo += np.matmul(dy[b].T, concat[b])
        dout_b += dy[b].sum(axis=0)
        dweighted = dconcat.reshape(q.shape[1], H, P).transpose(1, 0, 2)   # [H,Lq,P]
        ddrop = np.matmul(dweighted, proj_v[b].transpose(0, 2, 1))         # [H,Lq,Lk]
        dproj_v = np.matmul(attn_drop[b].transpose(0, 2, 1), dweighted)
        dalpha = dropout_backward_data(ddrop, None if softmax_mask is None else softmax_mask[b])
        dbeta = softmax_backward_data(alpha[b], dalpha, -1)     # grad wrt scale*scores
        dscores = scale * dbeta                                 # grad wrt raw q.k
        dproj_k = np.matmul(dscores.transpose(0, 2, 1), proj_q[b])
        dproj_q = np.matmul(dscores, proj_k[b])
        dv[b] = np.matmul(dproj_v, wv).sum(axis=0)
        dwv += np.matmul(dproj_v.transpose(0, 2, 1), v[b])
        din_b[2] += dproj_v.sum(axis=1)
        dk[b] = np.matmul(dproj_k, wk).sum(axis=0)
        dwk += np.matmul(dproj_k.transpose(0, 2, 1), k[b])
        din_b[1] += dproj_k.sum(axis=1)
        dq[b] = np.matmul(dproj_q, wq).sum(axis=0)
        dwq += np.matmul(dproj_q.transpose(0, 2, 1), q[b])
        din_b[0] += dproj_q.sum(axis=1)
        ddrop_.append(ddrop); dbeta_.append(dbeta)
    if self_attention:
        total = dq + dk + dv
        dq = dk = dv = total
    return dq, dk, dv, dwq, dwk, dwv, dwo, din_b, dout_b, ddrop_, dbeta_


# --------------------------------------------------------------------------
# encoder layer                               substation/transformer.py:176-285
# --------------------------------------------------------------------------

def encoder(x, attn_wq, attn_wk, attn_wv, attn_wo, attn_in_b, attn_out_b, attn_scale,
            norm1_scale, norm1_bias, norm2_scale, norm2_bias,
            linear1_w, linear1_b, linear2_w, linear2_b,
            softmax_mask=None, attn_dropout_mask=None, linear1_dropout_mask=None,
            ff_dropout_mask=None, activation='relu', ln_mode='rsqrt', attn_mask=None):
    """Post-LN encoder layer forward, transformer.py:176-209; with ``attn_mask``
    [L,L] (additive) it is the masked-self-attention layer ``decoder`` of
    transformer.py:443-476.  The backward pass does not see the mask
    (transformer.py:478-546 passes it on, attention.py:82-179 never reads it:
    a masked position has alpha = 0, hence no gradient).

    Masks: softmax_mask [B,H,L,L], attn_dropout_mask [B,L,E],
    linear1_dropout_mask [B,L,U], ff_dropout_mask [B,L,E]; None = no dropout.
    Returns a dict of every intermediate the backward pass and the parity tests
    need, keyed by the reference's variable names.
    """
    act = _ACT[activation][0]
    (attn, attn_concat, proj_q, proj_k, proj_v, alpha, attn_drop) = attn_forward(
        x, x, x, attn_wq, attn_wk, attn_wv, attn_wo, attn_in_b, attn_out_b, attn_scale,
        softmax_mask, attn_mask)
    attn_resid = dropout(attn, attn_dropout_mask) + x
    normed1, norm1_mean, norm1_std, norm1_normed = layer_norm(
        attn_resid, norm1_scale, norm1_bias, ln_mode=ln_mode)
    ff1_linear = linear(normed1, linear1_w, bias=linear1_b)
    ff1 = dropout(act(ff1_linear), linear1_dropout_mask)
    ff = linear(ff1, linear2_w, bias=linear2_b)
    ff_resid = dropout(ff, ff_dropout_mask) + normed1
    normed2, norm2_mean, norm2_std, norm2_normed = layer_norm(
        ff_resid, norm2_scale, norm2_bias, ln_mode=ln_mode)
    return dict(y=normed2, attn=attn, attn_concat=attn_concat, attn_proj_q=proj_q,
                attn_proj_k=proj_k, attn_proj_v=proj_v, attn_scaled_scores=alpha,
                attn_drop=attn_drop, norm1_mean=norm1_mean, norm1_std=norm1_std,
                norm1_normed=norm1_normed, norm2_mean=norm2_mean, norm2_std=norm2_std,
                norm2_normed=norm2_normed, ff=ff, ff_resid=ff_resid, ff1=ff1,
                ff1_linear=ff1_linear, normed1=normed1, attn_resid=attn_resid)


def encoder_backward(x, dy, fwd, attn_wq, attn_wk, attn_wv, attn_wo, attn_scale,
                     norm1_scale, norm2_scale, linear1_w, linear1_b, linear2_w, linear2_b,
                     softmax_mask=None, attn_dropout_mask=None, linear1_dropout_mask=None,
                     ff_dropout_mask=None, activation='relu', relu_gate=None):
    """Backward data + weights, transformer.py:212-285.  ``fwd`` = encoder()'s dict.

    ``relu_gate`` ([B,L,U] of {0,1}) replaces ``ff1_linear > 0`` in the ReLU
    derivative.  ReLU's derivative is discontinuous at 0, so a forward value that
    an fp16 path rounds to the other side of 0 flips one gradient element by its
    full size; parity tests of a reduced-precision device path therefore feed
    the gate the device saved (its stored LIN1 > 0), exactly as they feed the
    dropout masks.  The reference's kernel reads the gate from its stored LIN1 as
    well (pytorch_module/block_bdrlb.cuh:72).

    Returns a dict: dx, dattn_wq/wk/wv/wo, dattn_in_b (q,k,v order), dattn_out_b,
    dnorm{1,2}_{scale,bias}, dlinear{1,2}_{w,b}, plus the intermediate gradients
    the device path materialises (names in the comments).
    """
    act_bwd = _ACT[activation][1]
    f = fwd
    dff_resid = layer_norm_backward_data(                                    # DRESID2
        f['ff_resid'], dy, f['norm2_mean'], f['norm2_std'], norm2_scale)
    dnorm2_scale, dnorm2_bias = layer_norm_backward_weights(dy, f['norm2_normed'])
    dff = dropout_backward_data(dff_resid, ff_dropout_mask)                  # DLIN2
    dff1 = linear_backward_data(f['ff1'], linear2_w, dff)                    # DDROP2
    dlinear2_w, dlinear2_b = linear_backward_weights(f['ff1'], linear2_w, dff, bias=linear2_b)
    dff1_act = dropout_backward_data(dff1, linear1_dropout_mask)
    if relu_gate is not None and activation == 'relu':
        dff1_linear = relu_gate * dff1_act
    else:
        dff1_linear = act_bwd(f['ff1_linear'], dff1_act)                     # DLIN1
    dnormed1_linear = linear_backward_data(f['normed1'], linear1_w, dff1_linear)  # DLIN1_LINW1
    dlinear1_w, dlinear1_b = linear_backward_weights(
        f['normed1'], linear1_w, dff1_linear, bias=linear1_b)
    dnormed1 = dff_resid + dnormed1_linear
    dattn_resid = layer_norm_backward_data(                                  # DRESID1
        f['attn_resid'], dnormed1, f['norm1_mean'], f['norm1_std'], norm1_scale)
    dnorm1_scale, dnorm1_bias = layer_norm_backward_weights(dnormed1, f['norm1_normed'])
    dattn = dropout_backward_data(dattn_resid, attn_dropout_mask)            # DATT
    (dx_attn, _, _, dwq, dwk, dwv, dwo, din_b, dout_b, ddrop, dbeta) = attn_backward(
        x, x, x, attn_wq, attn_wk, attn_wv, attn_wo, attn_scale, dattn,
        f['attn_concat'], f['attn_proj_q'], f['attn_proj_k'], f['attn_proj_v'],
        f['attn_scaled_scores'], f['attn_drop'], softmax_mask, self_attention=True)
    dx = dattn_resid + dx_attn
    return dict(dx=dx, dattn_wq=dwq, dattn_wk=dwk, dattn_wv=dwv, dattn_wo=dwo,
                dattn_in_b=din_b, dattn_out_b=dout_b,
                dnorm1_scale=dnorm1_scale, dnorm1_bias=dnorm1_bias,
                dnorm2_scale=dnorm2_scale, dnorm2_bias=dnorm2_bias,
                dlinear1_w=dlinear1_w, dlinear1_b=dlinear1_b,
                dlinear2_w=dlinear2_w, dlinear2_b=dlinear2_b,
                dff_resid=dff_resid, dff=dff, dff1=dff1, dff1_linear=dff1_linear,
                dnormed1_linear=dnormed1_linear, dnormed1=dnormed1,
                dattn_resid=dattn_resid, dattn=dattn, dx_attn=dx_attn,
                dattn_drop=ddrop, dbeta=dbeta)


# --------------------------------------------------------------------------
# Mapping to the device module's tensor names (canonical dim order)
# pytorch_module/run_encoder.py:155-184, 207-325; encoder.cu:87-299
# --------------------------------------------------------------------------

#: canonical dim order of every named tensor of the device path
CANONICAL = dict(
    X='BJI', SB2='BJI',
    WKQV='QPHI', BKQV='QPH', WO='IPH', BO='I', S1='I', B1='I', LINB1='U', LINW1='IU',
    S2='I', B2='I', LINB2='I', LINW2='UI',
    KKQQVV='QPHBJ', WKKWQQWVV='QPHBJ', BETA='HBJK', ALPHA='HBJK', ATTN_DROP_MASK='HBJK',
    ATTN_DROP='HBJK', GAMMA='PHBJ', ATT='BJI', DROP1MASK='BJI', SB1='BJI', SB1_LINW1='BJU',
    DROP2='BJU', LIN1='BJU', DROP2_LINW2='BJI', LIN2='BJI', LN2='BJI', LN2STD='BJ',
    LN2DIFF='BJI', DROP2MASK='BJU', DROP3MASK='BJI', LN1='BJI', LN1STD='BJ', LN1DIFF='BJI',
    DLN2='BJI', DRESID2='BJI', DLIN2='BJI', DDROP2='BJU', DLIN1='BJU', DLIN1_LINW1='BJI',
    DLN1='BJI', DRESID1='BJI', DATT='BJI', DXATT='BJI', DGAMMA='PHBJ', DATTN_DROP='HBJK',
    DBETA='HBJK', DKKQQVV='QPHBJ',
)


def module_params_to_numpy(p):
    """Device-module parameters (canonical dim order, see CANONICAL) -> the
    argument set of ``encoder``; run_encoder.py:155-184.  Stack index of
    WKQV/BKQV is 0=K, 1=Q, 2=V (encoder.cu:93-99); in_b is (q,k,v)."""
    wkqv = np.einsum('QPHI->QHPI', p['WKQV'])
    bkqv = np.einsum('QPH->QHP', p['BKQV'])
    I = p['WO'].shape[0]
    wo = np.einsum('IPH->IHP', p['WO']).reshape(I, -1)
    return dict(
        attn_wq=wkqv[1], attn_wk=wkqv[0], attn_wv=wkqv[2], attn_wo=wo,
        attn_in_b=np.stack((bkqv[1], bkqv[0], bkqv[2])), attn_out_b=p['BO'],
        norm1_scale=p['S1'], norm1_bias=p['B1'], norm2_scale=p['S2'], norm2_bias=p['B2'],
        linear1_w=np.ascontiguousarray(p['LINW1'].T), linear1_b=p['LINB1'],
        linear2_w=np.ascontiguousarray(p['LINW2'].T), linear2_b=p['LINB2'])


def run_named(params, X, DY, masks=None, activation='relu', ln_mode='rsqrt', relu_gate=None,
              attn_mask=None):
    """Forward + backward with device-module naming.

    params: dict name -> array in canonical dim order (CANONICAL); X, DY [B,J,I];
    masks: dict with optional ATTN_DROP_MASK [H,B,J,K], DROP1MASK [B,J,I],
    DROP2MASK [B,J,U], DROP3MASK [B,J,I] of {0,1}.  Returns dict name -> array in
    canonical dim order for SB2, every forward/backward intermediate of the
    device path, DX and the 12 parameter gradients ('D'+name).
    """
    masks = masks or {}
    a = module_params_to_numpy(params)
    H, P = a['attn_wq'].shape[0], a['attn_wq'].shape[1]
    scale = 1.0 / np.sqrt(P)
    sm = masks.get('ATTN_DROP_MASK')
    sm_b = None if sm is None else np.einsum('HBJK->BHJK', sm)
    mk = dict(softmax_mask=sm_b, attn_dropout_mask=masks.get('DROP1MASK'),
              linear1_dropout_mask=masks.get('DROP2MASK'), ff_dropout_mask=masks.get('DROP3MASK'))
    f = encoder(X, a['attn_wq'], a['attn_wk'], a['attn_wv'], a['attn_wo'], a['attn_in_b'],
                a['attn_out_b'], scale, a['norm1_scale'], a['norm1_bias'], a['norm2_scale'],
                a['norm2_bias'], a['linear1_w'], a['linear1_b'], a['linear2_w'], a['linear2_b'],
                activation=activation, ln_mode=ln_mode, attn_mask=attn_mask, **mk)
    g = encoder_backward(X, DY, f, a['attn_wq'], a['attn_wk'], a['attn_wv'], a['attn_wo'], scale,
                         a['norm1_scale'], a['norm2_scale'], a['linear1_w'], a['linear1_b'],
                         a['linear2_w'], a['linear2_b'], activation=activation,
                         relu_gate=relu_gate, **mk)
    B, J, I = X.shape
    out = {}
    pq = np.stack(f['attn_proj_q']); pk = np.stack(f['attn_proj_k']); pv = np.stack(f['attn_proj_v'])
    kkqqvv = np.stack([np.einsum('BHJP->PHBJ', t) for t in (pk, pq, pv)])       # Q=0:K,1:Q,2:V
    out['KKQQVV'] = kkqqvv
    out['WKKWQQWVV'] = kkqqvv - params['BKQV'][:, :, :, None, None]
    alpha = np.einsum('BHJK->HBJK', np.stack(f['attn_scaled_scores']))
    out['ALPHA'] = alpha
    out['ATTN_DROP'] = np.einsum('BHJK->HBJK', np.stack(f['attn_drop']))
    out['BETA'] = scale * np.einsum('BHJK->HBJK', np.matmul(pq, np.swapaxes(pk, -1, -2)))
    out['GAMMA'] = np.einsum('BJHP->PHBJ', np.stack(f['attn_concat']).reshape(B, J, H, P))
    out['ATT'] = f['attn']                                   # biased, as stored in place
    out['LN1DIFF'] = f['attn_resid'] - f['norm1_mean']
    out['LN1STD'] = (1.0 / f['norm1_std'])[..., 0]
    out['LN1'] = f['norm1_normed']
    out['SB1'] = f['normed1']
    out['LIN1'] = f['ff1_linear']
    out['SB1_LINW1'] = f['ff1_linear'] - params['LINB1']
    out['DROP2'] = f['ff1']
    out['LIN2'] = f['ff']
    out['DROP2_LINW2'] = f['ff'] - params['LINB2']
    out['LN2DIFF'] = f['ff_resid'] - f['norm2_mean']
    out['LN2STD'] = (1.0 / f['norm2_std'])[..., 0]
    out['LN2'] = f['norm2_normed']
    out['SB2'] = f['y']
    # backward intermediates
    out['DLN2'] = DY * params['S2']
    out['DRESID2'] = g['dff_resid']
    out['DLIN2'] = g['dff']
    out['DDROP2'] = g['dff1']
    out['DLIN1'] = g['dff1_linear']
    out['DLIN1_LINW1'] = g['dnormed1_linear']
    out['DLN1'] = g['dnormed1'] * params['S1']
    out['DRESID1'] = g['dattn_resid']
    out['DATT'] = g['dattn']
    out['DXATT'] = g['dx_attn']
    out['DATTN_DROP'] = np.einsum('BHJK->HBJK', np.stack(g['dattn_drop']))
    out['DBETA'] = np.einsum('BHJK->HBJK', np.stack(g['dbeta']))
    dgamma = np.matmul(g['dattn'], a['attn_wo']).reshape(B, J, H, P)
    out['DGAMMA'] = np.einsum('BJHP->PHBJ', dgamma)
    # DKKQQVV from the bias-gradient-free definition: grads of the projections
    dbeta_b = np.stack(g['dbeta'])
    # (batched matmul: the same sums as 'BHJK,BHKP->BHJP', 'BHJK,BHJP->BHKP' twice)
    dpq = scale * np.matmul(dbeta_b, pk)
    dpk = scale * np.matmul(np.swapaxes(dbeta_b, -1, -2), pq)
    dpv = np.matmul(np.swapaxes(np.stack(f['attn_drop']), -1, -2), np.einsum('BJHP->BHJP', dgamma))
    out['DKKQQVV'] = np.stack([np.einsum('BHJP->PHBJ', t) for t in (dpk, dpq, dpv)])
    # outputs and parameter gradients
    out['DX'] = g['dx']
    dw = np.stack((g['dattn_wk'], g['dattn_wq'], g['dattn_wv']))               # [Q,H,P,I]
    out['DWKQV'] = np.einsum('QHPI->QPHI', dw)
    db = np.stack((g['dattn_in_b'][1], g['dattn_in_b'][0], g['dattn_in_b'][2]))  # [Q,H,P]
    out['DBKQV'] = np.einsum('QHP->QPH', db)
    out['DWO'] = np.einsum('IHP->IPH', g['dattn_wo'].reshape(I, H, P))
    out['DBO'] = g['dattn_out_b']
    out['DS1'] = g['dnorm1_scale']; out['DB1'] = g['dnorm1_bias']
    out['DS2'] = g['dnorm2_scale']; out['DB2'] = g['dnorm2_bias']
    out['DLINB1'] = g['dlinear1_b']; out['DLINW1'] = np.ascontiguousarray(g['dlinear1_w'].T)
    out['DLINB2'] = g['dlinear2_b']; out['DLINW2'] = np.ascontiguousarray(g['dlinear2_w'].T)
    return out


# --------------------------------------------------------------------------
# Closed forms of the fused operators, one per device kernel
# pytorch_module/benchmark.py compare_with_reference methods
# --------------------------------------------------------------------------

def op_softmax(beta, mask, scale=1.0):
    """benchmark.py:379-393. -> (ALPHA, ATTN_DROP)."""
    alpha = softmax(scale * beta, -1)
    return alpha, alpha * mask


def op_bad(inp, bias, mask, activation='relu'):
    """benchmark.py:453-468. -> (LIN, OUT)."""
    lin = inp + bias
    return lin, _ACT[activation][0](lin) * mask


def op_bdrln(inp, resid, lin_bias, scale, bias, mask, eps=1e-5):
    """benchmark.py:549-569 (with the kernel's eps, block_bdrln.cuh:258).
    -> (LIN, ISTD, DIFF, NORMED, OUT)."""
    lin = inp + lin_bias
    r = lin * mask + resid
    mean = r.mean(axis=-1, keepdims=True)
    istd = 1.0 / np.sqrt(r.var(axis=-1) + eps)
    diff = r - mean
    normed = diff * istd[..., None]
    return lin, istd, diff, normed, normed * scale + bias


def op_blnrd(dout, istd, diff, mask):
    """benchmark.py:642-661. -> (D_LN_IN, D_DROP_IN)."""
    n = dout.shape[-1]
    a = dout * istd[..., None]
    b = (dout.sum(axis=-1) * istd / n)[..., None]
    c = ((dout * diff).sum(axis=-1) * istd ** 3 / n)[..., None] * diff
    d = a - b - c
    return d, d * mask


def op_bsb(inp, scale, dout):
    """benchmark.py:728-744. -> (DIN, DSCALE, DBIAS)."""
    return dout * scale, np.einsum('bji,bji->i', dout, inp), np.einsum('bji->i', dout)


def op_ebsb(inp, scale, dout1, dout2, dlinear):
    """benchmark.py:980-995. -> (DIN, DSCALE, DBIAS, DLINEAR_BIAS)."""
    d = dout1 + dout2
    return (d * scale, np.einsum('bji,bji->i', d, inp), np.einsum('bji->i', d),
            np.einsum('bji->i', dlinear))


def op_bdrlb(ddrop, mask, lin, activation='relu'):
    """benchmark.py:814-827 (GELU via transformer.py:17-28). -> (DLINEAR, DBIAS)."""
    d = _ACT[activation][1](lin, ddrop * mask)
    return d, np.einsum('bju->u', d)


def op_bs(alpha, mask, ddrop, scale=1.0):
    """benchmark.py:891-903. -> DBETA (times ``scale`` when the softmax scaled)."""
    dalpha = ddrop * mask
    return scale * alpha * (dalpha - np.sum(alpha * dalpha, axis=-1, keepdims=True))


def op_aib(w, bias):
    """benchmark.py:1163-1176 on the stacked tensor: w [Q,P,H,B,J] + bias [Q,P,H]."""
    return w + bias[..., None, None]


def op_baib(d):
    """benchmark.py:1242-1258 on the stacked tensor: [Q,P,H,B,J] -> [Q,P,H]."""
    return d.sum(axis=(-1, -2))


def op_baob(datt):
    """benchmark.py:1311-1325."""
    return datt.sum(axis=(0, 1))


def op_bei(dxatt, dresid1):
    """benchmark.py:1051-1062."""
    return dxatt + dresid1
