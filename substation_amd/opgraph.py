"""Operator graph of the encoder layer: which tensors each launch touches.

Counterpart of the ``OperatorDef`` tables of config_selection/ops.py:61-257 and
the linear order of config_selection/optimize.py:13-53, reduced to what a
search over layouts needs: per operator, the named tensors whose layouts decide
its running time.  Names are those of the layouts pickle
(pytorch_module/encoder.cu:87-299); ``SB2`` stands for both the layer output and
the incoming gradient DY, ``X`` for the input and the outgoing gradient DX
(config_selection/ops.py:265-289 ties them), and every weight gradient has the
layout of its weight.
"""
import itertools

from . import layouts as _lay

#: (operator, pass, tensors) in launch order
OPERATORS = [
    ('QKV-fused', 'fwd', ('X', 'WKQV', 'BKQV', 'WKKWQQWVV', 'KKQQVV')),
    ('aib', 'fwd', ('WKKWQQWVV', 'BKQV', 'KKQQVV')),
    ('attention', 'fwd', ('KKQQVV', 'BETA', 'ALPHA', 'ATTN_DROP_MASK', 'ATTN_DROP', 'GAMMA')),
    ('QKT+softmax', 'fwd', ('KKQQVV', 'BETA', 'ALPHA', 'ATTN_DROP_MASK', 'ATTN_DROP')),
    ('QKT', 'fwd', ('KKQQVV', 'BETA')),
    ('softmax', 'fwd', ('BETA', 'ALPHA', 'ATTN_DROP_MASK', 'ATTN_DROP')),
    ('gamma', 'fwd', ('KKQQVV', 'ATTN_DROP', 'GAMMA')),
    ('out', 'fwd', ('WO', 'GAMMA', 'ATT')),
    ('bdrln1', 'fwd', ('ATT', 'X', 'DROP1MASK', 'LN1DIFF', 'LN1', 'SB1', 'LN1STD')),
    ('lin1', 'fwd', ('SB1', 'LINW1', 'SB1_LINW1')),
    ('lin1+bad', 'fwd', ('SB1', 'LINW1', 'DROP2', 'LIN1')),                   # LIN1: GELU layers only
    ('bad', 'fwd', ('SB1_LINW1', 'LIN1', 'DROP2MASK', 'DROP2')),
    ('lin2', 'fwd', ('DROP2', 'LINW2', 'DROP2_LINW2')),
    ('bdrln2', 'fwd', ('DROP2_LINW2', 'SB1', 'LIN2', 'DROP3MASK', 'LN2DIFF', 'LN2', 'SB2', 'LN2STD')),
    ('bsb+blnrd1', 'bwd', ('LN2', 'SB2', 'DLN2', 'LN2STD', 'LN2DIFF', 'DROP3MASK', 'DRESID2', 'DLIN2')),
    ('bsb', 'bwd', ('LN2', 'SB2', 'DLN2')),
    ('blnrd1', 'bwd', ('DLN2', 'LN2STD', 'LN2DIFF', 'DROP3MASK', 'DRESID2', 'DLIN2')),
    ('dXlin2', 'bwd', ('DLIN2', 'LINW2', 'DDROP2')),
    ('dWlin2', 'bwd', ('DLIN2', 'DROP2', 'LINW2')),
    ('dXlin2+bdrlb', 'bwd', ('DLIN2', 'LINW2', 'DROP2', 'LIN1', 'DLIN1')),    # GELU: LIN1 and keep bits, not DROP2
    ('bdrlb', 'bwd', ('DDROP2', 'DROP2MASK', 'LIN1', 'DROP2', 'DLIN1')),      # ReLU: the gate is read off DROP2
    ('dXlin1+dWlin1', 'bwd', ('DLIN1', 'LINW1', 'DLIN1_LINW1', 'SB1')),
    # many tokens: the two weight gradients of the feed-forward block as a pair, dXlin1 alone
    ('dWlin1+dWlin2', 'bwd', ('DLIN1', 'SB1', 'LINW1', 'DLIN2', 'DROP2', 'LINW2')),
    ('dXlin1', 'bwd', ('DLIN1', 'LINW1', 'DLIN1_LINW1')),
    ('dWlin1', 'bwd', ('DLIN1', 'SB1', 'LINW1')),
    ('ebsb+blnrd2+baob', 'bwd', ('LN1', 'DRESID2', 'DLIN1_LINW1', 'DLIN2', 'DLN1', 'LN1STD', 'LN1DIFF',
                                 'DROP1MASK', 'DRESID1', 'DATT')),
    ('ebsb', 'bwd', ('LN1', 'DRESID2', 'DLIN1_LINW1', 'DLIN2', 'DLN1')),
    ('blnrd2', 'bwd', ('DLN1', 'LN1STD', 'LN1DIFF', 'DROP1MASK', 'DRESID1', 'DATT')),
    ('baob', 'bwd', ('DATT',)),
    ('dWout', 'bwd', ('GAMMA', 'DATT', 'WO')),
    ('dXout+dWout', 'bwd', ('WO', 'DATT', 'DGAMMA', 'GAMMA')),
    ('dXout', 'bwd', ('WO', 'DATT', 'DGAMMA')),
    ('attention-bwd-dQ', 'bwd', ('KKQQVV', 'GAMMA', 'DGAMMA', 'DATTN_DROP', 'ALPHA', 'ATTN_DROP_MASK', 'DBETA',
                                 'DKKQQVV')),
    ('attention-bwd-dKdV', 'bwd', ('KKQQVV', 'DGAMMA', 'ATTN_DROP', 'DATTN_DROP', 'ALPHA', 'ATTN_DROP_MASK',
                                   'DBETA', 'DKKQQVV')),
    ('dX1gamma+bs', 'bwd', ('KKQQVV', 'DGAMMA', 'DATTN_DROP', 'ALPHA', 'ATTN_DROP_MASK', 'DBETA')),
    ('dX1gamma', 'bwd', ('KKQQVV', 'DGAMMA', 'DATTN_DROP')),
    ('dX2gamma', 'bwd', ('DGAMMA', 'ATTN_DROP', 'DKKQQVV')),
    ('bs', 'bwd', ('ALPHA', 'ATTN_DROP_MASK', 'DATTN_DROP', 'DBETA')),
    ('dX1QKT', 'bwd', ('KKQQVV', 'DBETA', 'DKKQQVV')),
    ('dX2QKT', 'bwd', ('KKQQVV', 'DBETA', 'DKKQQVV')),
    ('dXQKV-fused+dWQKV-fused+dWout', 'bwd', ('WKQV', 'DKKQQVV', 'DXATT', 'DRESID1', 'X', 'GAMMA', 'DATT', 'WO')),
    ('dXQKV-fused+dWQKV-fused', 'bwd', ('WKQV', 'DKKQQVV', 'DXATT', 'DRESID1', 'X')),
    ('dXQKV-fused', 'bwd', ('WKQV', 'DKKQQVV', 'DXATT', 'DRESID1', 'X')),
    ('dWQKV-fused', 'bwd', ('X', 'DKKQQVV', 'WKQV')),
    ('baib', 'bwd', ('DKKQQVV', 'BKQV')),
    ('bei', 'bwd', ('DXATT', 'DRESID1', 'X')),
    # second stage of the pass's column sums when no launch before it had room for it
    ('colfinish', 'bwd', ()),
]
OP_TENSORS = {name: tensors for name, _, tensors in OPERATORS}

#: Launches that stand for one another: where the sizes and layouts allow it the
#: library runs the first entry of a group in place of the others (an addend
#: folded into a contraction's epilogue, several row kernels in one launch), so
#: which of them run depends on the layouts of the whole group's tensors.
ALTERNATIVES = [
    ('QKV-fused', 'aib'),
    # dWout runs inside the last launch of the pass when that has room for its tiles
    ('dXQKV-fused+dWQKV-fused+dWout', 'dXQKV-fused+dWQKV-fused', 'dXQKV-fused', 'dWQKV-fused', 'bei',
     'dXout+dWout', 'dXout', 'dWout', 'colfinish'),
    ('lin1+bad', 'lin1', 'bad'),
    # (dWlin2 waits for dWlin1 when the two run as a pair)
    ('dXlin2+bdrlb', 'dXlin2', 'bdrlb', 'dXlin1+dWlin1', 'dWlin1+dWlin2', 'dXlin1', 'dWlin1', 'dWlin2'),
    ('attention', 'QKT+softmax', 'QKT', 'softmax', 'gamma'),
    ('attention-bwd-dQ', 'attention-bwd-dKdV', 'dX2gamma', 'dX1gamma+bs', 'dX1gamma', 'bs', 'dX1QKT', 'dX2QKT',
     'baib'),
    ('bsb+blnrd1', 'bsb', 'blnrd1'),
    ('ebsb+blnrd2+baob', 'ebsb', 'blnrd2', 'baob'),
]

#: Tensors beyond its members' own that decide which members of a group run: the
#: attention kernels with the scores in registers need feature-contiguous
#: projections, outputs and gradients in both passes (one decision for both), and
#: whether dWout and the column-sum finish ride in the last launch of the backward
#: pass depends on that decision too.
_ATTENTION_DECIDERS = ('KKQQVV', 'GAMMA', 'DGAMMA', 'DKKQQVV')
GROUP_ALSO_DEPENDS = {
    'attention': _ATTENTION_DECIDERS,
    'attention-bwd-dQ': _ATTENTION_DECIDERS,
    'dXQKV-fused+dWQKV-fused+dWout': _ATTENTION_DECIDERS + ('BKQV',),
}

#: the 18 contractions (pytorch_module/encoder.cu:90-276; canonical list
#: tc_profiling/einsum_perms.py:367-394): name -> (A, B, C) operand names, where
#: KK/QQ/VV and DKK/DQQ/DVV are the Q-slices of the stacked tensors
EINSUMS = {
    'QKV-fused': ('X', 'WKQV', 'WKKWQQWVV'),
    'QKT': ('KK', 'QQ', 'BETA'),
    'gamma': ('VV', 'ATTN_DROP', 'GAMMA'),
    'out': ('WO', 'GAMMA', 'ATT'),
    'lin1': ('SB1', 'LINW1', 'SB1_LINW1'),
    'lin2': ('DROP2', 'LINW2', 'DROP2_LINW2'),
    'dXlin2': ('DLIN2', 'LINW2', 'DDROP2'),
    'dWlin2': ('DLIN2', 'DROP2', 'DLINW2'),
    'dXlin1': ('DLIN1', 'LINW1', 'DLIN1_LINW1'),
    'dWlin1': ('DLIN1', 'SB1', 'DLINW1'),
    'dWout': ('GAMMA', 'DATT', 'DWO'),
    'dXout': ('WO', 'DATT', 'DGAMMA'),
    'dX1gamma': ('VV', 'DGAMMA', 'DATTN_DROP'),
    'dX2gamma': ('DGAMMA', 'ATTN_DROP', 'DVV'),
    'dX1QKT': ('KK', 'DBETA', 'DQQ'),
    'dX2QKT': ('QQ', 'DBETA', 'DKK'),
    'dXQKV-fused': ('WKQV', 'DKKQQVV', 'DXATT'),
    'dWQKV-fused': ('X', 'DKKQQVV', 'DWKQV'),
}


def tensor_layouts(layouts):
    """name -> layout string for every tensor a layouts dict names."""
    return dict(list(layouts['params']) + list(layouts['forward_interm'])
                + list(layouts['backward_interm'])
                + [tuple(layouts['input']), tuple(layouts['output'])])


def operand_layouts(layouts):
    """tensor_layouts() plus the derived GEMM operands: weight gradients (layout of
    the weight) and the Q-slices, with the key/value sequence dim renamed J->K
    (pytorch_module/encoder.py:339-347)."""
    t = tensor_layouts(layouts)
    for k, v in list(layouts['params']):
        t['D' + k] = v
    kk, dkk = t['KKQQVV'][1:], t['DKKQQVV'][1:]
    t['QQ'] = kk
    t['KK'] = t['VV'] = kk.replace('J', 'K')
    t['DQQ'] = dkk
    t['DKK'] = t['DVV'] = dkk.replace('J', 'K')
    return t


def with_layouts(layouts, changes):
    """A copy of ``layouts`` with ``changes`` (name -> layout) applied."""
    def sub(pairs):
        return [(n, changes.get(n, l)) for n, l in pairs]
    out = dict(layouts)
    out['input'] = ('X', changes.get('X', layouts['input'][1]))
    out['output'] = ('SB2', changes.get('SB2', layouts['output'][1]))
    for key in ('params', 'forward_interm', 'backward_interm'):
        out[key] = sub(layouts[key])
    return out


def candidate_layouts(name):
    """Every layout a tensor may take: permutations of its dims, with the stacking
    dim first where pytorch_module/encoder.py:318-327 requires it."""
    dims = _lay.CANONICAL[name]
    if name in _lay._Q_FIRST:
        rest = dims.replace('Q', '')
        return ['Q' + ''.join(p) for p in itertools.permutations(rest)]
    return [''.join(p) for p in itertools.permutations(dims)]


def searchable_tensors():
    """Tensors with more than one possible layout, in pickle order."""
    names = ['X', 'SB2'] + _lay.PARAM_NAMES + _lay.FWD_NAMES + _lay.BWD_NAMES
    return [n for n in names if len(candidate_layouts(n)) > 1]
