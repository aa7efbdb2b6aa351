"""The entry point that allocates nothing, sub_op_ln_backward_static, through the C
ABI against sub_op_ln_backward: same kernels, partial sums in the library's static
device array instead of a buffer the handle allocates, results bit for bit the
same, on calls in a row that shrink (the array keeps the last call's contents)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(o, ext, seed):
    g = torch.Generator(device='cuda').manual_seed(seed)
    E = o.sizes['I']

    def t(layout, std=1.0):
        return o.empty(layout).normal_(0.0, std, generator=g)

    def v(mean=0.0, std=0.1):
        return torch.empty(E, dtype=torch.float16, device='cuda').normal_(mean, std, generator=g)

    d = dict(inp=t('BJI'), s=v(1.0), d1=t('BJI'), istd=t('BJ').abs_().add_(0.5), diff=t('BJI'),
             mask=(torch.rand(o.empty('BJI').shape, device='cuda', generator=g) >= 0.1).half())
    if ext:
        d.update(d2=t('BJI'), dl=t('BJI'))
    return d


def _run(o, d, ext, static):
    E = o.sizes['I']
    out = dict(g=o.empty('BJI'), a=o.empty('BJI'), b=o.empty('BJI'))
    for k in ('ds', 'db') + (('dlb', 'dob') if ext else ()):
        out[k] = torch.full((E,), float('nan'), dtype=torch.float16, device='cuda')
    kw = dict(static_scratch=static)
    if ext:
        kw.update(dout2=d['d2'], l_dout2='BJI', dlinear=d['dl'], l_dlinear='BJI', dlinear_bias=out['dlb'],
                  dout_bias=out['dob'])
    o.ln_backward(d['inp'], 'BJI', d['s'], d['d1'], 'BJI', d['istd'], 'BJ', d['diff'], 'BJI', d['mask'], 'BJI',
                  out['g'], 'BJI', out['a'], 'BJI', out['b'], 'BJI', out['ds'], out['db'], **kw)
    torch.cuda.synchronize()
    return out


def test_static_scratch_entry_point_matches_the_allocating_one_on_shrinking_calls():
    from substation_amd.ops import Ops
    # (B, L, H, E): rows of 1024 features in one launch; a smaller call; rows of 2048
    # features (the separate operators, each with its own partial rows); a tiny one
    cases = [((8, 512, 16, 1024), True), ((2, 128, 4, 256), True), ((2, 256, 16, 2048), True),
             ((4, 256, 16, 1024), False), ((1, 24, 2, 48), False)]
    handles = []
    for i, (dims, ext) in enumerate(cases):
        want_o, got_o = Ops(*dims), Ops(*dims)          # the second handle never allocates
        handles += [want_o, got_o]
        d = _inputs(want_o, ext, 100 + i)
        if i == 1:
            free_before = torch.cuda.mem_get_info()[0]
        got = _run(got_o, d, ext, static=True)
        if i == 1:
            # nothing was allocated on the device by that call (the first call has looked the array up)
            assert torch.cuda.mem_get_info()[0] == free_before
        want = _run(want_o, d, ext, static=False)
        for k in want:
            assert torch.isfinite(want[k].float()).all(), (dims, k)
            assert torch.equal(got[k], want[k]), (dims, ext, k)
