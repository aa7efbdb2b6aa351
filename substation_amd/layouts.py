"""Layout configurations ("the plugin config") of the encoder layer.

Schema (config_selection/optimize.py:443-493, consumed at
pytorch_module/encoder.py:56,81,111,117,229-376)::

    {'input': ('X', perm of BJI), 'output': ('SB2', perm of BJI),
     'params':          [(name, layout) x 12],
     'forward_interm':  [(name, layout) x 23],
     'backward_interm': [(name, layout) x 14],
     'special_dims': {...}, 'algorithms': {...}}

``special_dims`` (which dim each CUDA kernel vectorises / maps to threads) and
``algorithms`` (cuBLAS algorithm ids) are accepted and ignored: the HIP kernels
vectorise along whichever dim is contiguous and there is one GEMM kernel family.
"""
import pickle

PARAM_NAMES = ['WKQV', 'BKQV', 'WO', 'BO', 'S1', 'B1', 'LINB1', 'LINW1', 'S2', 'B2', 'LINB2', 'LINW2']
FWD_NAMES = ['KKQQVV', 'WKKWQQWVV', 'BETA', 'ALPHA', 'ATTN_DROP_MASK', 'ATTN_DROP', 'GAMMA', 'ATT',
             'DROP1MASK', 'SB1', 'SB1_LINW1', 'DROP2', 'LIN1', 'DROP2_LINW2', 'LIN2', 'LN2', 'LN2STD',
             'LN2DIFF', 'DROP2MASK', 'DROP3MASK', 'LN1', 'LN1STD', 'LN1DIFF']
BWD_NAMES = ['DLN2', 'DRESID2', 'DLIN2', 'DDROP2', 'DLIN1', 'DLIN1_LINW1', 'DLN1', 'DRESID1', 'DATT',
             'DXATT', 'DGAMMA', 'DATTN_DROP', 'DBETA', 'DKKQQVV']

#: canonical dimension order of every tensor (the set of dims each layout permutes)
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

_Q_FIRST = ('KKQQVV', 'DKKQQVV', 'WKKWQQWVV', 'BKQV', 'WKQV')   # encoder.py:318-327


def _pairs(text):
    return [tuple(tok.split(':')) for tok in text.split()]


def _algos(text):
    out = {}
    for tok in text.split():
        k, v = tok.split(':')
        out[k] = 'DEFAULT' if v == 'D' else 'ALGO' + v
    return out


def _make(inp, out, params, fwd, bwd, special='', algos=''):
    return {
        'input': ('X', inp), 'output': ('SB2', out),
        'params': _pairs(params), 'forward_interm': _pairs(fwd), 'backward_interm': _pairs(bwd),
        'special_dims': dict(_pairs(special)), 'algorithms': _algos(algos),
    }


def mi355x_layouts(name=None):
    """Configuration for MI355X (``name``: one of the two workloads the reference
    ships configurations for, or None for the default), read from the files the
    layout search (substation_amd.layout_search, the counterpart of
    config_selection/optimize.py) wrote from timings on the device:
    ``configs/layouts-mi355x-<name>.pickle``, same schema as the reference's
    pickles, decoded as plain data.  None is the configuration of
    'bert-b8-l512-h16-e1024'.

    What the search settles on: token-major activations with the feature
    dimension contiguous (every fused operator then moves 128-bit packs),
    projections stored [Q,B,J,H,P] and the attention output [B,J,H,P] so that
    QK^T, the output projection and both FFN products contract over a contiguous
    dimension of both operands, weights stored [out, in]; for B=96 L=128 the
    projection weight is stored [Q,I,H,P]."""
    if name not in (None, 'bert-b8-l512-h16-e1024', 'bert-b96-l128-h16-e1024'):
        raise KeyError(name)
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'configs',
                        f'layouts-mi355x-{name or "bert-b8-l512-h16-e1024"}.pickle')
    return load_layouts(path)


def reference_layouts(name):
    """The two configurations the reference ships
    (pytorch_module/layouts-bert-b8-l512-h16-e1024.pickle and
    pytorch_module/layouts-bert-b96-l128-h16-e1024.pickle), restated as literals."""
    params = 'WKQV:QPHI BKQV:QPH WO:IPH BO:I S1:I B1:I LINB1:U LINW1:IU S2:I B2:I LINB2:I '
    if name == 'bert-b8-l512-h16-e1024':
        return _make(
            'IBJ', 'IBJ', params + 'LINW2:UI',
            'KKQQVV:QPHBJ WKKWQQWVV:QPHBJ BETA:HBJK ALPHA:HBJK ATTN_DROP_MASK:HBJK ATTN_DROP:HBJK '
            'GAMMA:PHBJ ATT:BJI DROP1MASK:IBJ SB1:BJI SB1_LINW1:UBJ DROP2:UBJ LIN1:UBJ '
            'DROP2_LINW2:IBJ LIN2:BJI LN2:IBJ LN2STD:JB LN2DIFF:JBI DROP2MASK:UBJ DROP3MASK:JBI '
            'LN1:IBJ LN1STD:BJ LN1DIFF:JBI',
            'DLN2:IBJ DRESID2:IBJ DLIN2:IBJ DDROP2:UBJ DLIN1:UBJ DLIN1_LINW1:IBJ DLN1:IBJ '
            'DRESID1:BJI DATT:IBJ DXATT:BJI DGAMMA:PHBJ DATTN_DROP:HBJK DBETA:HBJK DKKQQVV:QPHBJ',
            'AIB_DT:J AIB_DV:J BAD_DT:J BAD_DV:U BAIB_DV:B BAIB_DW:J BAOB_DV:B BAOB_DW:J BDRLB_DV:J '
            'BDRLB_DW:J BDRLN1_DV:J BDRLN2_DV:J BEI_DT:J BEI_DV:I BLNRD1_DV:J BLNRD2_DV:J BSB_DV:J '
            'BSB_DW:J BS_DV:K EBSB_DV:J EBSB_DW:J SM_DV:K',
            'ATT:3 BETA:3 DATTN_DROP:3 DDROP2:3 DGAMMA:6 DKK:5 DLIN1_LINW1:D DLINW1:D DLINW2:D DQQ:0 '
            'DROP2_LINW2:D DVV:13 DWKQV:D DWO:D DXATT:D GAMMA:D SB1_LINW1:3 WKKWQQWVV:3')
    if name == 'bert-b96-l128-h16-e1024':
        return _make(
            'BJI', 'BJI', params + 'LINW2:IU',
            'KKQQVV:QHBPJ WKKWQQWVV:QPHBJ BETA:HBJK ALPHA:HBJK ATTN_DROP_MASK:HBJK ATTN_DROP:HBJK '
            'GAMMA:PHBJ ATT:BJI DROP1MASK:BJI SB1:BJI SB1_LINW1:BJU DROP2:BJU LIN1:BJU '
            'DROP2_LINW2:BJI LIN2:JBI LN2:JBI LN2STD:BJ LN2DIFF:BJI DROP2MASK:BJU DROP3MASK:BJI '
            'LN1:BJI LN1STD:BJ LN1DIFF:BJI',
            'DLN2:JBI DRESID2:IBJ DLIN2:BJI DDROP2:UBJ DLIN1:UBJ DLIN1_LINW1:IBJ DLN1:IBJ '
            'DRESID1:IBJ DATT:IBJ DXATT:BJI DGAMMA:PHBJ DATTN_DROP:HBJK DBETA:HBJK DKKQQVV:QPHBJ',
            'AIB_DT:J AIB_DV:B BAD_DT:U BAD_DV:U BAIB_DV:J BAIB_DW:B BAOB_DV:J BAOB_DW:B BDRLB_DV:U '
            'BDRLB_DW:J BDRLN1_DV:I BDRLN2_DV:I BEI_DT:I BEI_DV:J BLNRD1_DV:J BLNRD2_DV:J BSB_DV:I '
            'BSB_DW:B BS_DV:K EBSB_DV:J EBSB_DW:J SM_DV:K',
            'ATT:3 BETA:1 DATTN_DROP:9 DDROP2:D DGAMMA:D DKK:2 DLIN1_LINW1:6 DLINW1:D DLINW2:D DQQ:10 '
            'DROP2_LINW2:6 DVV:10 DWKQV:D DWO:D DXATT:6 GAMMA:2 SB1_LINW1:3 WKKWQQWVV:D')
    raise KeyError(name)


def validate(layouts):
    """Checks the schema and the constraints of encoder.py:318-327."""
    for key in ('input', 'output', 'params', 'forward_interm', 'backward_interm'):
        if key not in layouts:
            raise ValueError(f'layouts: missing key {key!r}')
    groups = (('params', PARAM_NAMES), ('forward_interm', FWD_NAMES), ('backward_interm', BWD_NAMES))
    for key, names in groups:
        got = [n for n, _ in layouts[key]]
        if sorted(got) != sorted(names):
            raise ValueError(f'layouts[{key!r}] must list exactly {names}, got {got}')
    allt = dict(list(layouts['params']) + list(layouts['forward_interm'])
                + list(layouts['backward_interm']) + [tuple(layouts['input']), tuple(layouts['output'])])
    if layouts['input'][0] != 'X' or layouts['output'][0] != 'SB2':
        raise ValueError("layouts: input must be ('X', ...) and output ('SB2', ...)")
    for name, lay in allt.items():
        if sorted(lay) != sorted(CANONICAL[name]):
            raise ValueError(f'layout of {name} must be a permutation of {CANONICAL[name]}, got {lay}')
    for name in _Q_FIRST:
        if allt[name][0] != 'Q':
            raise ValueError(f'layout of {name} must start with Q, got {allt[name]}')
    return layouts


def _read_data_pickle(data):
    """Decodes a pickle that holds only dict / list / tuple / str / int / bool /
    None.  The byte stream is walked with ``pickletools.genops`` (a disassembler)
    and rebuilt by the small stack machine below; opcodes that name, import or
    call anything (GLOBAL, REDUCE, BUILD, NEWOBJ, ...) are rejected, so nothing
    from the file can execute."""
    import pickletools
    stack, marks, memo = [], [], {}
    mark = object()

    def pop_mark():
        i = len(stack) - 1 - stack[::-1].index(mark)
        items = stack[i + 1:]
        del stack[i:]
        return items

    for op, arg, _ in pickletools.genops(data):
        n = op.name
        if n in ('PROTO', 'FRAME'):
            continue
        elif n == 'STOP':
            break
        elif n == 'MARK':
            stack.append(mark)
        elif n == 'EMPTY_DICT':
            stack.append({})
        elif n == 'EMPTY_LIST':
            stack.append([])
        elif n == 'EMPTY_TUPLE':
            stack.append(())
        elif n in ('BINUNICODE', 'SHORT_BINUNICODE', 'BINUNICODE8', 'UNICODE', 'BININT', 'BININT1',
                   'BININT2', 'INT', 'LONG1', 'BINFLOAT'):
            stack.append(arg)
        elif n == 'NONE':
            stack.append(None)
        elif n in ('NEWTRUE', 'NEWFALSE'):
            stack.append(n == 'NEWTRUE')
        elif n in ('MEMOIZE',):
            memo[len(memo)] = stack[-1]
        elif n in ('BINPUT', 'LONG_BINPUT', 'PUT'):
            memo[arg] = stack[-1]
        elif n in ('BINGET', 'LONG_BINGET', 'GET'):
            stack.append(memo[arg])
        elif n == 'TUPLE':
            stack.append(tuple(pop_mark()))
        elif n in ('TUPLE1', 'TUPLE2', 'TUPLE3'):
            k = int(n[-1])
            items = stack[-k:]
            del stack[-k:]
            stack.append(tuple(items))
        elif n == 'APPEND':
            v = stack.pop(); stack[-1].append(v)
        elif n == 'APPENDS':
            items = pop_mark(); stack[-1].extend(items)
        elif n == 'SETITEM':
            v = stack.pop(); k = stack.pop(); stack[-1][k] = v
        elif n == 'SETITEMS':
            items = pop_mark()
            for i in range(0, len(items), 2):
                stack[-1][items[i]] = items[i + 1]
        elif n == 'DICT':
            items = pop_mark()
            stack.append({items[i]: items[i + 1] for i in range(0, len(items), 2)})
        elif n == 'LIST':
            stack.append(list(pop_mark()))
        else:
            raise pickle.UnpicklingError(
                f'layouts file uses pickle opcode {n}; only plain dict/list/tuple/str data is allowed')
    if len(stack) != 1:
        raise pickle.UnpicklingError('malformed layouts pickle')
    return stack[0]


def load_layouts(path):
    """Reads a layouts pickle written by the reference's
    config_selection/optimize.py:443-493 (or by save_layouts)."""
    with open(path, 'rb') as f:
        data = f.read()
    return validate(_read_data_pickle(data))


def save_layouts(layouts, path):
    with open(path, 'wb') as f:
        pickle.dump(validate(layouts), f)


def shape_of(layout, sizes):
    return tuple(sizes[d] for d in layout)


def sizes_map(batch_size, max_seq_len, num_heads, embedding_size, intermediate_size=None):
    """pytorch_module/encoder.py:43-53."""
    return {'Q': 3, 'B': batch_size, 'S': max_seq_len, 'H': num_heads,
            'P': embedding_size // num_heads, 'I': embedding_size,
            'U': intermediate_size or 4 * embedding_size, 'J': max_seq_len, 'K': max_seq_len}
