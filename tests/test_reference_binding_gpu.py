"""The reference's own way of calling the library, executed on the GPU: the ctypes
binding that the integration notes at the repository root give a maintainer of
pytorch_module/encoder.py to put in place of `_compile_module` is taken from
there verbatim, and the four exports of pytorch_module/encoder.cu:304-318 are then
driven as pytorch_module/encoder.py:71-139 drives them: `init()`, positional
`encoder_forward` (1 + 37 pointers) and `encoder_backward` (1 + 64 pointers) in
the order of the lists of the layouts dict, `destroy()`.  Results against the
NumPy oracle, masks against the seeded Philox oracle."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from oracle import encoder_ref as ref
from oracle import philox_ref as ph
from tests.helpers import assert_close, from_layout, h16

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def option_b_source():
    text = open(os.path.join(ROOT, 'INTEGRATION.md')).read()
    section = text[text.index('## Option B'):]
    return re.search(r'```python\n(.*?)```', section, re.S).group(1)


def test_option_b_snippet_is_python():
    src = option_b_source()
    compile(src, 'INTEGRATION.md', 'exec')
    assert 'encoder_forward.argtypes' in src and 'encoder_backward.argtypes' in src and 'init_cfg' in src


@pytest.mark.gpu
@pytest.mark.parametrize('which', ['bert-b8-l512-h16-e1024', 'mi355x'])
def test_positional_exports_through_the_reference_binding(which):
    from substation_amd import _lib, layouts as L
    lay = L.reference_layouts(which) if which != 'mi355x' else L.mi355x_layouts()
    B, S, H, E, p = 2, 128, 2, 128, 0.1
    sizes = L.sizes_map(B, S, H, E, 4 * E)
    sizes['S'] = S                                  # the reference's name for the sequence length
    ns = {}
    exec(option_b_source().replace("'libsubstation_amd.so'", repr(_lib.LIB_PATH)), ns)
    compile_module = ns['_compile_module']
    compile_module = getattr(compile_module, '__func__', compile_module)
    lib = compile_module(sizes, 'half', lay, p, p, p, p, False, 'unused')
    handle = lib.init()                             # encoder.py:71
    assert handle
    lib.sub_last_error.restype = ctypes.c_char_p

    rng = np.random.default_rng(3)
    params_np, weights = {}, []
    for name, layout in lay['params']:              # encoder.py:56-60: one tensor per entry, in layout order
        canon = ref.CANONICAL[name]
        shape = tuple(sizes[d] for d in canon)
        v = (1 + 0.1 * rng.normal(size=shape)) if name in ('S1', 'S2') else \
            (0.1 if len(canon) == 1 or name == 'BKQV' else 0.05) * rng.normal(size=shape)
        params_np[name] = h16(v)
        weights.append(torch.from_numpy(
            np.transpose(params_np[name], [canon.index(d) for d in layout]).copy()).half().cuda())
    X_np = h16(rng.normal(size=(B, S, E))); DY_np = h16(rng.normal(size=(B, S, E)))
    lx, ly = lay['input'][1], lay['output'][1]
    X = torch.from_numpy(np.transpose(X_np, ['BJI'.index(d) for d in lx]).copy()).half().cuda()
    DY = torch.from_numpy(np.transpose(DY_np, ['BJI'.index(d) for d in ly]).copy()).half().cuda()
    empty = lambda layout: torch.empty(tuple(sizes[d] for d in layout), device='cuda', dtype=torch.float16)
    # encoder.py:75-93
    Y = empty(ly)
    fwd = [empty(l) for _, l in lay['forward_interm']]
    rc = lib.encoder_forward(handle, X.data_ptr(), *(t.data_ptr() for t in weights),
                             *(t.data_ptr() for t in fwd), Y.data_ptr())
    assert rc == 0, lib.sub_last_error()
    # encoder.py:106-130
    DX = empty(lx)
    bwd = [empty(l) for _, l in lay['backward_interm']]
    grads = [torch.empty_like(w) for w in weights]
    rc = lib.encoder_backward(handle, DY.data_ptr(), *(t.data_ptr() for t in grads),
                              *(t.data_ptr() for t in bwd), *(t.data_ptr() for t in weights),
                              *(t.data_ptr() for t in fwd), X.data_ptr(), DX.data_ptr())
    assert rc == 0, lib.sub_last_error()
    torch.cuda.synchronize()
    lib.destroy(handle)

    got = {'SB2': from_layout(Y, 'BJI', ly), 'DX': from_layout(DX, 'BJI', lx)}
    for (name, layout), g in zip(lay['params'], grads):
        got['D' + name] = from_layout(g, ref.CANONICAL[name], layout)
    U = sizes['U']
    masks = {name: ph.dropout_mask(shape, p, 0, site, step=0, dtype=np.float64)       # the snippet's seed is 0
             for name, shape, site in (('ATTN_DROP_MASK', (H, B, S, S), 0), ('DROP1MASK', (B, S, E), 1),
                                       ('DROP2MASK', (B, S, U), 2), ('DROP3MASK', (B, S, E), 3))}
    names = [n for n, _ in lay['forward_interm']]
    layouts_f = dict(lay['forward_interm'])
    # (the intermediates lie in the order sub_tensor_layout names: the configured one, or, for a configuration
    # with feature-major activations, the library's own)
    held = ctypes.create_string_buffer(16)
    lib.sub_tensor_layout.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p]
    assert lib.sub_tensor_layout(handle, b'DROP2', held) == 0, lib.sub_last_error()
    held = held.value.decode()
    assert held == ('BJU' if which != 'mi355x' else layouts_f['DROP2'])
    drop2 = from_layout(fwd[names.index('DROP2')].reshape(-1).view([sizes[d] for d in held]), 'BJU', held)
    assert (drop2[masks['DROP2MASK'] == 0] == 0).all()
    # by default the residual dropout masks travel as one bit per element, canonical order, in
    # the first B*J*I/8 bytes of their buffers (SUB_OPT_PACKED_MASKS)
    for name in ('DROP1MASK', 'DROP3MASK'):
        raw = fwd[names.index(name)].contiguous().view(torch.uint8).reshape(-1)[:B * S * E // 8].cpu().numpy()
        bits = np.unpackbits(raw, bitorder='little').reshape(B, S, E)
        assert (bits == masks[name]).all(), name
    # ReLU layer (the reference's only activation): the gate the backward pass read, as in the other layer tests
    want = ref.run_named(params_np, X_np, DY_np, masks, 'relu', relu_gate=(drop2 > 0).astype(np.float64))
    for name in ('SB2', 'DX') + tuple('D' + n for n, _ in lay['params']):
        assert_close(got[name], want[name], tol=1e-2, name=name)
