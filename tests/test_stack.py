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
