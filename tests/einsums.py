"""The 18 tensor contractions of the layer (pytorch_module/encoder.cu:90-276,
canonical list tc_profiling/einsum_perms.py:367-394) as
(name, A tensor, B tensor, C tensor, scaled-by-1/sqrt(P)), with the dims of each
operand as a function of its layout, including the K/V renaming J->K
(pytorch_module/encoder.py:339-347)."""

EINSUMS = [
    ('QKV-fused', 'X', 'WKQV', 'WKKWQQWVV', False),
    ('QKT', 'KK', 'QQ', 'BETA', True),
    ('gamma', 'VV', 'ATTN_DROP', 'GAMMA', False),
    ('out', 'WO', 'GAMMA', 'ATT', False),
    ('lin1', 'SB1', 'LINW1', 'SB1_LINW1', False),
    ('lin2', 'DROP2', 'LINW2', 'DROP2_LINW2', False),
    ('dXlin2', 'DLIN2', 'LINW2', 'DDROP2', False),
    ('dWlin2', 'DLIN2', 'DROP2', 'DLINW2', False),
    ('dXlin1', 'DLIN1', 'LINW1', 'DLIN1_LINW1', False),
    ('dWlin1', 'DLIN1', 'SB1', 'DLINW1', False),
    ('dWout', 'GAMMA', 'DATT', 'DWO', False),
    ('dXout', 'WO', 'DATT', 'DGAMMA', False),
    ('dX1gamma', 'VV', 'DGAMMA', 'DATTN_DROP', False),
    ('dX2gamma', 'DGAMMA', 'ATTN_DROP', 'DVV', False),
    ('dX1QKT', 'KK', 'DBETA', 'DQQ', True),
    ('dX2QKT', 'QQ', 'DBETA', 'DKK', True),
    ('dXQKV-fused', 'WKQV', 'DKKQQVV', 'DXATT', False),
    ('dWQKV-fused', 'X', 'DKKQQVV', 'DWKQV', False),
]


def operand_layouts(layouts):
    """name -> layout string for every GEMM operand of a layouts dict."""
    t = dict(list(layouts['params']) + list(layouts['forward_interm'])
             + list(layouts['backward_interm']) + [tuple(layouts['input']), tuple(layouts['output'])])
    for k, v in list(layouts['params']):
        t['D' + k] = v
    kk = t['KKQQVV'][1:]
    dkk = t['DKKQQVV'][1:]
    t['QQ'] = kk; t['KK'] = kk.replace('J', 'K'); t['VV'] = kk.replace('J', 'K')
    t['DQQ'] = dkk; t['DKK'] = dkk.replace('J', 'K'); t['DVV'] = dkk.replace('J', 'K')
    return t
