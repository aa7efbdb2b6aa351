"""Layers chained into a stack: persistent workspaces, canonical checkpoints."""
import numpy as np
import pytest
import torch

from tests.helpers import assert_close

SEED = 77


def _small_stack(lay, **kw):
    from substation_amd import EncoderStack
    return EncoderStack(2, 2, 128, 2, 128, lay, torch.float16, 0.1, 0.1, 0.1, 0.1, activation='gelu', seed=SEED, **kw)


def test_canonical_state_dict_is_independent_of_the_layouts():
    """A checkpoint written by a stack built with one set of layouts loads into a
    stack built with another; element (q,p,h,i) of a weight stays element (q,p,h,i)."""
    from substation_amd import layouts as L
    a = _small_stack(L.mi355x_layouts())
    b = _small_stack(L.reference_layouts('bert-b8-l512-h16-e1024'))
    sd = a.state_dict()
    for name, lay in a.layers[0].layouts['params']:
        canon = L.CANONICAL[name]
        t = sd['layers.0.' + name]
        assert tuple(t.shape) == tuple(a.layers[0].sizes[d] for d in canon), name
        perm = [lay.index(d) for d in canon]
        assert torch.equal(t, getattr(a.layers[0], name).detach().permute(perm))
    b.load_state_dict(sd)
    for la, lb in zip(a.layers, b.layers):
        for (name, lay_a), (_, lay_b) in zip(la.layouts['params'], lb.layouts['params']):
            canon = L.CANONICAL[name]
            pa = getattr(la, name).detach().permute([lay_a.index(d) for d in canon])
            pb = getattr(lb, name).detach().permute([lay_b.index(d) for d in canon])
            assert torch.equal(pa, pb), name
    # a layer without the option keeps the reference's behaviour: parameters as stored
    from substation_amd import Encoder
    e = Encoder('unused', 2, 128, 2, 128, L.reference_layouts('bert-b8-l512-h16-e1024'), torch.float16,
                0.1, 0.1, 0.1, 0.1)
    assert all(tuple(v.shape) == tuple(getattr(e, k).shape) for k, v in e.state_dict().items())


def test_stack_needs_matching_input_and_output_layouts():
    from substation_amd import EncoderStack, layouts as L
    lay = dict(L.mi355x_layouts())
    lay['output'] = ('SB2', 'JBI')
    with pytest.raises(ValueError, match='stack'):
        EncoderStack(2, 2, 128, 2, 128, lay, torch.float16, 0.1, 0.1, 0.1, 0.1)


@pytest.mark.gpu
def test_stack_equals_separately_applied_layers_iteration_after_iteration():
    """A stack with persistent, shared workspaces and compact attention buffers
    gives, bit for bit, what independent layers with per-call allocations give
    (same parameters, same dropout streams), on the first iteration and on the
    later ones that reuse the buffers; the workspaces do not grow."""
    from substation_amd import Encoder, layouts as L
    lay = L.mi355x_layouts()
    stack = _small_stack(lay).cuda()
    plain = [Encoder('unused', 2, 128, 2, 128, lay, torch.float16, 0.1, 0.1, 0.1, 0.1, activation='gelu',
                     seed=SEED + i).cuda() for i in range(2)]
    with torch.no_grad():
        for layer, ref in zip(stack.layers, plain):
            for p, q in zip(layer.parameters(), ref.parameters()):
                p.mul_(0.2)
                q.copy_(p)
    g = torch.Generator().manual_seed(3)
    held = None
    for it in range(3):
        X = torch.randn(2, 128, 128, generator=g).half().cuda()
        DY = torch.randn(2, 128, 128, generator=g).half().cuda()
        xs = X.clone().requires_grad_(True)
        xp = X.clone().requires_grad_(True)
        stack.zero_grad(); [m.zero_grad() for m in plain]
        ys = stack(xs)
        ys.backward(DY)
        h = xp
        for m in plain:
            h = m(h)
        h.backward(DY)
        torch.cuda.synchronize()
        assert torch.equal(ys, h) and torch.equal(xs.grad, xp.grad), it
        for layer, ref in zip(stack.layers, plain):
            for (n, p), q in zip(layer.named_parameters(), ref.parameters()):
                assert torch.equal(p.grad, q.grad), (it, n)
        if held is None:
            held = stack.workspace_bytes()
            assert held > 0
        assert stack.workspace_bytes() == held


@pytest.mark.gpu
def test_persistent_workspace_refuses_a_backward_pass_whose_inputs_were_overwritten():
    from substation_amd import layouts as L
    stack = _small_stack(L.mi355x_layouts()).cuda()
    X = torch.randn(2, 128, 128).half().cuda().requires_grad_(True)
    y1 = stack(X)
    y2 = stack(X)
    y2.sum().backward()
    with pytest.raises(RuntimeError, match='persistent_workspace'):
        y1.sum().backward()


@pytest.mark.gpu
def test_checkpoint_moves_between_layout_configurations():
    """The same canonical checkpoint under the MI355X default layouts and under the
    reference's shipped configuration: same function (other kernels, other
    summation orders: compared at the parity bound)."""
    from substation_amd import layouts as L
    a = _small_stack(L.mi355x_layouts()).cuda()
    with torch.no_grad():
        for p in a.parameters():
            p.mul_(0.2)
    lay_b = L.reference_layouts('bert-b8-l512-h16-e1024')
    b = _small_stack(lay_b).cuda()
    b.load_state_dict(a.state_dict())
    a.set_rng(SEED, 0); b.set_rng(SEED, 0)
    g = torch.Generator().manual_seed(4)
    X = torch.randn(2, 128, 128, generator=g).half()                      # [B, J, I]
    xa = X.cuda().requires_grad_(True)
    to_b = ['BJI'.index(d) for d in lay_b['input'][1]]
    xb = X.permute(to_b).contiguous().cuda().requires_grad_(True)
    ya, yb = a(xa), b(xb)
    from_b = [lay_b['output'][1].index(d) for d in 'BJI']
    assert_close(yb.detach().permute(from_b).float().cpu().numpy(), ya.detach().float().cpu().numpy(), tol=1e-2, name='Y')
    # and back: the same output gradient through both stacks (under the reference's configuration every layer
    # runs in the library's own orders and copies what crosses its boundary)
    DY = torch.randn(2, 128, 128, generator=g).half()
    ya.backward(DY.cuda())
    to_b_out = ['BJI'.index(d) for d in lay_b['output'][1]]
    yb.backward(DY.permute(to_b_out).contiguous().cuda())
    from_b_in = [lay_b['input'][1].index(d) for d in 'BJI']
    assert_close(xb.grad.permute(from_b_in).float().cpu().numpy(), xa.grad.float().cpu().numpy(), tol=1e-2, name='DX')


@pytest.mark.gpu
@pytest.mark.parametrize('act', ['gelu', 'relu'])
def test_stack_matches_the_oracle_applied_layer_by_layer(act):
    """Two stacked layers against the NumPy oracle applied twice: layer i draws its
    four dropout masks from the Philox stream of seed + i, layer 1's input is layer
    0's output, and layer 0's backward pass starts from layer 1's DX.  Output, DX
    and the 12 gradients of both layers to 1e-2 (config_selection/ops.py:265-270
    ties X and SB2 so that layers chain).  Shared backward workspace, compact
    attention and activation buffers, persistent forward workspaces: all on."""
    from oracle import encoder_ref as ref
    from oracle import philox_ref as ph
    from substation_amd import EncoderStack, layouts as L
    from tests.helpers import from_layout, h16
    from tests.test_encoder_gpu import OUTPUTS, _compare
    B, Ls, H, E, p = 2, 256, 4, 256, 0.1
    lay = L.mi355x_layouts()
    stack = EncoderStack(2, B, Ls, H, E, lay, torch.float16, p, p, p, p, activation=act, seed=SEED).cuda()
    stack.set_rng(SEED, 0)
    rng = np.random.default_rng(41)
    sz = stack.layers[0].sizes
    params = []
    for layer in stack.layers:
        pn = {}
        for name, layout in lay['params']:
            canon = ref.CANONICAL[name]
            shape = tuple(sz[d] for d in canon)
            v = (1 + 0.1 * rng.normal(size=shape)) if name in ('S1', 'S2') else \
                (0.1 if len(canon) == 1 or name == 'BKQV' else 0.05) * rng.normal(size=shape)
            pn[name] = h16(v)
            with torch.no_grad():
                getattr(layer, name).copy_(torch.from_numpy(
                    np.transpose(pn[name], [canon.index(d) for d in layout]).copy()).half())
        params.append(pn)
    X_np = h16(rng.normal(size=(B, Ls, E))); DY_np = h16(rng.normal(size=(B, Ls, E)))
    X = torch.from_numpy(X_np).half().cuda().requires_grad_(True)
    Y = stack(X)
    Y.backward(torch.from_numpy(DY_np).half().cuda())
    torch.cuda.synchronize()
    U = sz['U']
    masks, gates = [], []
    fwd_names = [n for n, _ in lay['forward_interm']]
    for i, layer in enumerate(stack.layers):
        masks.append({name: ph.dropout_mask(shape, p, SEED + i, site, step=0, dtype=np.float64)
                      for name, shape, site in (('ATTN_DROP_MASK', (H, B, Ls, Ls), 0), ('DROP1MASK', (B, Ls, E), 1),
                                                ('DROP2MASK', (B, Ls, U), 2), ('DROP3MASK', (B, Ls, E), 3))})
        gate = None
        if act == 'relu':      # the gate the device's backward pass used: DROP2 > 0 (see run_layer_default)
            drop2 = layer._workspace['forward_interm'][fwd_names.index('DROP2')]
            gate = (from_layout(drop2, 'BJU', 'BJU') > 0).astype(np.float64)
        gates.append(gate)
    # oracle: forward through both layers, then backward through both
    f0 = ref.run_named(params[0], X_np, DY_np, masks[0], act, relu_gate=gates[0])
    # what layer 1 sees is layer 0's fp16-rounded output
    x1 = h16(f0['SB2'])
    w1 = ref.run_named(params[1], x1, DY_np, masks[1], act, relu_gate=gates[1])
    w0 = ref.run_named(params[0], X_np, h16(w1['DX']), masks[0], act, relu_gate=gates[0])
    got1 = {'SB2': from_layout(Y, 'BJI', 'BJI'), 'DX': w1['DX']}      # layer 1's DX is internal to the stack
    got0 = {'SB2': f0['SB2'], 'DX': from_layout(X.grad, 'BJI', 'BJI')}  # layer 0's output likewise
    for got, layer in ((got0, stack.layers[0]), (got1, stack.layers[1])):
        for name, layout in lay['params']:
            got['D' + name] = from_layout(getattr(layer, name).grad, ref.CANONICAL[name], layout)
    _compare(w1, got1, names=OUTPUTS)
    _compare(w0, got0, names=OUTPUTS)
    # different streams per layer: the two layers' masks differ
    assert (masks[0]['DROP1MASK'] != masks[1]['DROP1MASK']).any()


@pytest.mark.gpu
def test_captured_stack_replays_match_eager_runs():
    """Forward + backward of a two-layer stack recorded in one HIP graph (after an
    eager warm-up that makes the one-time allocations) and replayed with eager work
    in between: every replay equals the eager run at the same dropout step bit for
    bit, with the step counters in device memory so that replays draw new masks."""
    from substation_amd import EncoderStack, layouts as L
    lay = L.mi355x_layouts()
    B, Ls, H, E = 2, 128, 4, 256

    def make(device_step):
        torch.manual_seed(0)
        st = EncoderStack(2, B, Ls, H, E, lay, torch.float16, 0.1, 0.1, 0.1, 0.1, seed=SEED).cuda()
        with torch.no_grad():
            for q in st.parameters():
                q.mul_(0.1)
        st.set_rng(SEED, 0)
        counters = [layer.use_device_step() for layer in st.layers] if device_step else None
        return st, counters

    g0 = torch.Generator().manual_seed(9)
    X = torch.randn(B, Ls, E, generator=g0).half().cuda().requires_grad_(True)
    DY = torch.randn(B, Ls, E, generator=g0).half().cuda()

    def collect(st, Y):
        return [Y.detach().clone(), X.grad.clone()] + [q.grad.clone() for q in st.parameters()]

    def clear(st):
        X.grad = None
        for q in st.parameters():
            q.grad = None

    st, counters = make(True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            clear(st)
            st(X).backward(DY)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert all(int(c.item()) == 2 for c in counters)
    clear(st)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        Y = st(X)
        Y.backward(DY)
    replays = []
    for r in range(3):
        graph.replay()
        torch.cuda.synchronize()
        replays.append(collect(st, Y))
        assert all(int(c.item()) == 3 + r for c in counters)
        _ = (torch.randn(1 << 20, device='cuda') * 2).sum().item()
    eager, _ = make(False)
    for r in range(3):
        eager.set_rng(SEED, 2 + r)
        clear(eager)
        Yr = eager(X)
        Yr.backward(DY)
        torch.cuda.synchronize()
        for a, b in zip(replays[r], collect(eager, Yr)):
            assert torch.equal(a, b), f'replay {r} differs from the eager run at step {2 + r}'
    assert not torch.equal(replays[0][0], replays[1][0])
