"""Benchmark of the fused encoder layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2|3|4|5] [--layouts mi355x|ref]

A step is one forward + one backward pass of a single encoder layer over one
batch of synthetic input (the protocol of pytorch_module/run_encoder.py:345-383).
The default workload is BERT-large B=8 L=512 H=16 E=1024 fp16 with the four
dropouts at p=0.1.  The timed region -- W untimed steps, then K steps between
two synchronisations on the host clock -- is run twice: as the process finds
the device (`cold_start_ms_per_step`) and again behind 150 ms of the same
steps (`value`: a device left idle for a few tens of milliseconds is slow for
the next 10-20 ms of work, and the figure to compare with the reference's
medians over 1000 iterations is the steady one; --preheat-ms 0 makes `value`
the cold figure).  Prints ONE JSON line: ms per layer, the per-launch
roofline measured live with HIP events on the launch stream, and the CPU
baseline (the NumPy oracle on the bench workload and on the reference's own
CPU-sized case).  --config 2 times the fused operators on their own (softmax
and its backward at [H=16,B=8,J=512,K=512], and every other memory-bound
operator at the default workload's shapes) and prints their line instead.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12        # B/s, MI355X HBM3E
MFMA_PEAK_F16 = 2.5e15   # FLOP/s, MI355X dense fp16
PEAK_MHZ = 2400.0        # the engine clock that peak is quoted at
V100_MS = 6.71           # reference README.md:23, V100-SXM2, same layer and sizes

CONFIGS = {
    3: dict(B=8, L=512, H=16, E=1024, act='relu', w_std=0.02, b_std=0.02,
            name='configs[2]: BERT-large encoder layer fwd+bwd B=8 L=512 H=16 E=1024 P=64 FF=4096 '
                 'post-LN ReLU fp16, 4 dropouts p=0.1 seeded'),
    4: dict(B=96, L=128, H=16, E=1024, act='relu', w_std=0.02, b_std=0.02,
            name='configs[3]: BERT-large encoder layer fwd+bwd B=96 L=128 H=16 E=1024 fp16'),
    5: dict(B=4, L=2048, H=32, E=4096, act='gelu', w_std=0.01, b_std=0.0,
            name='configs[4]: wide encoder layer fwd+bwd B=4 L=2048 H=32 E=4096 P=128 FF=16384 GELU fp16'),
}

TRAFFIC_PROFILE = os.path.join(ROOT, 'profiles', 'encoder_layer_b8_l512_hbm_traffic.txt')


def measured_traffic(path=TRAFFIC_PROFILE):
    """launch name -> HBM-side bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by a
    copy of known size) read from the tracked rocprofv3 summary of this workload; {} when the
    file is not there.  Table rows are `name fetch-MiB write-MiB total-MiB algorithmic-MiB ratio`."""
    out = {}
    try:
        lines = open(path).read().splitlines()
    except OSError:
        return out
    for line in lines:
        f = line.split()
        if len(f) != 6:
            continue
        try:
            nums = [float(x) for x in f[1:]]
        except ValueError:
            continue
        out[f[0]] = int(round(nums[2] * (1 << 20)))
    return out


GEMM_OPS = ('QKV-fused', 'QKT', 'gamma', 'out', 'lin1', 'lin2', 'dXlin2', 'dWlin2', 'dXlin1', 'dWlin1',
            'dWout', 'dXout', 'dX1gamma', 'dX2gamma', 'dX1QKT', 'dX2QKT', 'dXQKV-fused', 'dWQKV-fused')


#: the orders the library runs a feature-major configuration in (SUB_OPT_PRIVATE_LAYOUTS): weights that are
#: copied across the boundary when the configuration names another order
OWN_WEIGHT_ORDERS = {'WKQV': 'QHPI', 'BKQV': 'QHP', 'WO': 'IHP', 'LINW1': 'UI', 'LINW2': 'IU'}


def staged_elements(layouts, B, L, H, E):
    """Elements copied across the boundary per pass when the library runs a configuration in its own orders:
    (input or output [B,J,I] tensors, weights) -- 0, 0 for a configuration whose activations are all token-major."""
    acts = [layouts['input'][1], layouts['output'][1]] + [l for _, l in layouts['forward_interm']] \
        + [l for _, l in layouts['backward_interm']]
    own = {'BJI', 'BJU', 'HBJK', 'QBJHP', 'BJHP', 'BJ'}
    if all(l in own for l in acts):
        return 0, 0
    U, P = 4 * E, E // H
    numel = {'WKQV': 3 * E * E, 'BKQV': 3 * E, 'WO': E * E, 'LINW1': E * U, 'LINW2': E * U}
    w = sum(numel[n] for n, l in layouts['params'] if n in OWN_WEIGHT_ORDERS and l != OWN_WEIGHT_ORDERS[n])
    return B * L * E, w


def algorithmic_work(B, L, H, E, relu_from_output=True, packed_masks=True, skip_unread=True, staged=(0, 0)):
    """Per operator: ('hbm', bytes) or ('mfma', flops, bytes).  Bytes = each big
    tensor read once + written once in fp16; flops = 2*batch*M*N*K.
    relu_from_output: the ReLU layer as it runs by default -- bad writes only its
    output (one [B,J,U] tensor in, one out) and bdrlb reads the gate off that output
    (two in, one out); otherwise both move four.
    packed_masks: the two residual dropout masks as one bit per element (the default):
    1/16 of a [B,J,I] tensor where bdrln writes and the LayerNorm backward reads them.
    skip_unread: the [B,J,I] output that nothing reads afterwards is not written by
    bdrln (input + bias) and by the one-launch LayerNorm backward (the scaled gradient)."""
    U, P = 4 * E, E // H
    bji, bju, hbjk, q = B * L * E, B * L * U, H * B * L * L, 3 * B * L * E
    mk = bji // 8 if packed_masks else bji * 2           # bytes of one residual dropout mask
    un = 0 if skip_unread else bji * 2                   # bytes of an output nothing reads
    w = {
        'aib': ('hbm', 2 * q * 2), 'softmax': ('hbm', 4 * hbjk * 2), 'bs': ('hbm', 4 * hbjk * 2),
        'bdrln1': ('hbm', 5 * bji * 2 + mk + un), 'bdrln2': ('hbm', 5 * bji * 2 + mk + un),
        'blnrd1': ('hbm', 4 * bji * 2 + mk), 'blnrd2': ('hbm', 4 * bji * 2 + mk),
        'bsb': ('hbm', 3 * bji * 2), 'ebsb': ('hbm', 5 * bji * 2), 'baob': ('hbm', bji * 2),
        'bei': ('hbm', 3 * bji * 2), 'bad': ('hbm', (2 if relu_from_output else 4) * bju * 2),
        'bdrlb': ('hbm', (3 if relu_from_output else 4) * bju * 2),
        'baib': ('hbm', q * 2),
        # second stage of the column sums when it runs as a launch of its own: fp32 partial rows
        # in, a few vectors out (not one of the reference's operators: no algorithmic bytes)
        'colfinish': ('hbm', 0),
        # single-launch forms: the scaled gradient is written but not read back
        # (bsb + blnrd1 - one [B,J,I] read; ebsb + blnrd2 + baob - two reads)
        # (moved: the extended launch does not read DLIN2, whose column sum the plain launch took along)
        'bsb+blnrd1': ('hbm', 5 * bji * 2 + mk + un),
        'ebsb+blnrd2+baob': ('hbm', (6 if packed_masks or skip_unread else 7) * bji * 2 + mk + un),
        # scores formed in place: the score tensor itself is neither written nor read
        # (QKT + softmax: Q, K in, three score-sized tensors out; dX1gamma + bs: dO, V
        # and two score-sized tensors in, one out)
        'QKT+softmax': ('hbm', (3 * hbjk + 2 * bji) * 2), 'dX1gamma+bs': ('hbm', (3 * hbjk + 2 * bji) * 2),
    }
    # copies across the boundary of a configuration that runs in the library's own orders: read + write
    sa, sw = staged
    w['relayout-in'] = ('hbm', 4 * (sa + sw))
    w['relayout-out'] = ('hbm', 4 * sa)
    w['relayout-in-bwd'] = ('hbm', 4 * sa)
    w['relayout-in-again'] = ('hbm', 4 * (sa + sw))
    w['relayout-out-bwd'] = ('hbm', 4 * (sa + sw))
    tok = B * L
    proj = (2 * tok * 3 * E * E, 2 * (tok * E + 3 * E * E + 3 * tok * E))
    attn = (2 * H * B * L * L * P, 2 * (2 * tok * E + hbjk))
    outp = (2 * tok * E * E, 2 * (2 * tok * E + E * E))
    ffn = (2 * tok * E * U, 2 * (tok * E + E * U + tok * U))
    for n in ('QKV-fused', 'dXQKV-fused', 'dWQKV-fused'):
        w[n] = ('mfma',) + proj
    for n in ('QKT', 'gamma', 'dX1gamma', 'dX2gamma', 'dX1QKT', 'dX2QKT'):
        w[n] = ('mfma',) + attn
    # attention with the scores in registers: 2 / 3 / 4 products of the size of QKT
    # (the backward launches form the scores again); bytes: the projections, the
    # output or gradients, one keep bit per score
    # (a fourth entry: the products the algorithm has -- QKT, gamma forward; dX1gamma, dX1QKT and
    # dX2gamma, dX2QKT backward -- without the scores and their gradient formed a second time)
    w['attention'] = ('mfma', 2 * attn[0], 2 * 4 * bji + hbjk // 8, 2 * attn[0])
    w['attention-bwd-dQ'] = ('mfma', 3 * attn[0], 2 * 6 * bji + hbjk // 8, 2 * attn[0])
    w['attention-bwd-dKdV'] = ('mfma', 4 * attn[0], 2 * 6 * bji + hbjk // 8, 2 * attn[0])
    # two products in one launch
    w['dXlin1+dWlin1'] = ('mfma', 2 * ffn[0], 2 * ffn[1])
    w['dWlin1+dWlin2'] = ('mfma', 2 * ffn[0], 2 * ffn[1])
    w['dXQKV-fused+dWQKV-fused'] = ('mfma', 2 * proj[0], 2 * proj[1])
    w['dXout+dWout'] = ('mfma', 2 * outp[0], 2 * outp[1])
    # the last launch of the backward pass with dWout's tiles in the places it leaves free
    w['dXQKV-fused+dWQKV-fused+dWout'] = ('mfma', 2 * proj[0] + outp[0], 2 * proj[1] + outp[1])
    # lin1 with bias, ReLU and dropout in its epilogue: the product's flops, SB1 and LINW1 in, DROP2 out
    # the ReLU gate travels as one bit per element of DROP2: written by lin1's epilogue, read by dXlin2's
    w['lin1+bad'] = ('mfma', ffn[0], ffn[1] + tok * U // 8)
    w['dXlin2+bdrlb'] = ('mfma', ffn[0], ffn[1] + tok * U // 8)
    for n in ('out', 'dWout', 'dXout'):
        w[n] = ('mfma',) + outp
    for n in ('lin1', 'lin2', 'dXlin2', 'dWlin2', 'dXlin1', 'dWlin1'):
        w[n] = ('mfma',) + ffn
    return w


def make_encoder(cfg, layouts_name, profiling=False, seed=0x5EED):
    import torch
    from substation_amd import Encoder, layouts as L
    shipped = {(8, 512): 'bert-b8-l512-h16-e1024', (96, 128): 'bert-b96-l128-h16-e1024'}
    lay = (L.mi355x_layouts(shipped.get((cfg['B'], cfg['L'])) if cfg['E'] == 1024 else None)
           if layouts_name == 'mi355x'
           else L.reference_layouts('bert-b8-l512-h16-e1024' if cfg['L'] >= 512 else 'bert-b96-l128-h16-e1024'))
    enc = Encoder('unused', cfg['B'], cfg['L'], cfg['H'], cfg['E'], lay, torch.float16,
                  0.1, 0.1, 0.1, 0.1, profiling=profiling, activation=cfg['act'], seed=seed)
    g = torch.Generator().manual_seed(1000 + cfg['E'])
    with torch.no_grad():
        for name, _ in lay['params']:
            p = getattr(enc, name)
            t = torch.randn(p.shape, generator=g, dtype=torch.float32)
            if name in ('S1', 'S2'):
                t = torch.ones_like(t)
            elif name in ('B1', 'B2'):
                t = torch.zeros_like(t)
            elif p.dim() == 1 or name == 'BKQV':
                t = cfg['b_std'] * t
            else:
                t = cfg['w_std'] * t
            p.copy_(t)
    enc = enc.cuda()
    sz = enc.sizes
    shape = tuple(sz[d] for d in lay['input'][1])
    X = torch.randn(shape, generator=g, dtype=torch.float32).half().cuda().requires_grad_(True)
    DY = torch.randn(shape, generator=g, dtype=torch.float32).half().cuda()
    return enc, X, DY


def cpu_baseline(cfg, budget_s=20.0):
    """The NumPy oracle (a port of substation/transformer.py + attention.py with
    the reference's per-sample np.matmul structure) on the benchmark's own
    workload shape, forward + backward with p=0.1 masks fed, in fp32 (NumPy has
    no fp16 BLAS).  Bounded: one warm-up, then whole layers until about
    budget_s seconds are used (3 to 40 of them).  A workload whose single layer
    would exceed the budget is sampled at batch 1 and scaled by the batch size."""
    import numpy as np
    from oracle import encoder_ref as ref
    B, L, H, E, act = cfg['B'], cfg['L'], cfg['H'], cfg['E'], cfg['act']
    U, P = 4 * E, E // H
    flops = 3 * (2 * B * L * (4 * E * E + 2 * E * U) + 4 * B * H * L * L * P)
    scale_b = 1
    if flops > 4e12:               # > ~10 s per layer on a 16-core host
        scale_b, B = B, 1
    rng = np.random.default_rng(1001)
    f32 = np.float32
    params = dict(
        WKQV=(0.02 * rng.normal(size=(3, P, H, E))).astype(f32), BKQV=np.zeros((3, P, H), f32),
        WO=(0.02 * rng.normal(size=(E, P, H))).astype(f32), BO=np.zeros(E, f32),
        S1=np.ones(E, f32), B1=np.zeros(E, f32), LINB1=np.zeros(U, f32),
        LINW1=(0.02 * rng.normal(size=(E, U))).astype(f32), S2=np.ones(E, f32), B2=np.zeros(E, f32),
        LINB2=np.zeros(E, f32), LINW2=(0.02 * rng.normal(size=(U, E))).astype(f32))
    X = rng.normal(size=(B, L, E)).astype(f32); DY = rng.normal(size=(B, L, E)).astype(f32)
    a = ref.module_params_to_numpy(params)
    scale = f32(1.0 / np.sqrt(P))
    keep = lambda shape: (rng.random(shape, dtype=f32) >= f32(0.1)).astype(f32)     # {0,1} masks, p = 0.1
    mk = dict(softmax_mask=keep((B, H, L, L)), attn_dropout_mask=keep((B, L, E)),
              linear1_dropout_mask=keep((B, L, U)), ff_dropout_mask=keep((B, L, E)))

    def one():
        f = ref.encoder(X, a['attn_wq'], a['attn_wk'], a['attn_wv'], a['attn_wo'], a['attn_in_b'],
                        a['attn_out_b'], scale, a['norm1_scale'], a['norm1_bias'], a['norm2_scale'],
                        a['norm2_bias'], a['linear1_w'], a['linear1_b'], a['linear2_w'], a['linear2_b'],
                        activation=act, **mk)
        ref.encoder_backward(X, DY, f, a['attn_wq'], a['attn_wk'], a['attn_wv'], a['attn_wo'], scale,
                             a['norm1_scale'], a['norm2_scale'], a['linear1_w'], a['linear1_b'],
                             a['linear2_w'], a['linear2_b'], activation=act, **mk)

    one()
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 40):
        t0 = time.perf_counter(); one(); times.append(time.perf_counter() - t0)
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get('num_threads', 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = int(os.environ.get('OMP_NUM_THREADS', '1'))
    what = (f'B={B} L={L} H={H} E={E} FF={U} {act} fp32 fwd+bwd, p=0.1 masks fed, median of {len(times)} layers '
            f'({sum(times):.1f} s)')
    if scale_b > 1:
        what += f'; one sample of the batch of {scale_b}, time multiplied by {scale_b}'
    return {
        'value': round(statistics.median(times) * 1e3 * scale_b, 1), 'unit': 'ms/layer', 'cores': threads,
        'kind': 'port',
        'sample': f'NumPy oracle on the bench workload shape {what}; host has {os.cpu_count()} logical CPUs',
        'config1': cpu_baseline_config1(),
    }


def cpu_baseline_config1(warmups=3, runs=10):
    """BASELINE configs[0], the reference's own CPU-runnable case: B=2 L=128 H=12 E=768 P=64
    FF=3072 post-LN ReLU fp32, X, dY ~ N(0,1), weights N(0,0.02), biases 0, gamma=1, beta=0,
    p=0.1 masks from the seed; forward + backward, time.perf_counter, 3 warm-ups, median of 10.
    Two implementations side by side: the NumPy oracle (per-sample np.matmul structure of
    substation/transformer.py:176-285) and torch.nn.TransformerEncoderLayer on the CPU (what
    test/test_transformer_torch.py:280-340 checks the NumPy path against)."""
    import numpy as np
    import torch
    from oracle import encoder_ref as ref
    B, L, H, E = 2, 128, 12, 768
    U, P = 4 * E, E // H
    rng = np.random.default_rng(1001)
    f32 = np.float32
    params = dict(
        WKQV=(0.02 * rng.normal(size=(3, P, H, E))).astype(f32), BKQV=np.zeros((3, P, H), f32),
        WO=(0.02 * rng.normal(size=(E, P, H))).astype(f32), BO=np.zeros(E, f32),
        S1=np.ones(E, f32), B1=np.zeros(E, f32), LINB1=np.zeros(U, f32),
        LINW1=(0.02 * rng.normal(size=(E, U))).astype(f32), S2=np.ones(E, f32), B2=np.zeros(E, f32),
        LINB2=np.zeros(E, f32), LINW2=(0.02 * rng.normal(size=(U, E))).astype(f32))
    X = rng.normal(size=(B, L, E)).astype(f32); DY = rng.normal(size=(B, L, E)).astype(f32)
    a = ref.module_params_to_numpy(params)
    scale = f32(1.0 / np.sqrt(P))
    keep = lambda shape: (rng.random(shape, dtype=f32) >= f32(0.1)).astype(f32)
    mk = dict(softmax_mask=keep((B, H, L, L)), attn_dropout_mask=keep((B, L, E)),
              linear1_dropout_mask=keep((B, L, U)), ff_dropout_mask=keep((B, L, E)))

    def numpy_step():
        f = ref.encoder(X, a['attn_wq'], a['attn_wk'], a['attn_wv'], a['attn_wo'], a['attn_in_b'],
                        a['attn_out_b'], scale, a['norm1_scale'], a['norm1_bias'], a['norm2_scale'],
                        a['norm2_bias'], a['linear1_w'], a['linear1_b'], a['linear2_w'], a['linear2_b'],
                        activation='relu', **mk)
        ref.encoder_backward(X, DY, f, a['attn_wq'], a['attn_wk'], a['attn_wv'], a['attn_wo'], scale,
                             a['norm1_scale'], a['norm2_scale'], a['linear1_w'], a['linear1_b'],
                             a['linear2_w'], a['linear2_b'], activation='relu', **mk)

    torch.manual_seed(1001)
    layer = torch.nn.TransformerEncoderLayer(E, H, U, dropout=0.1, activation='relu')     # post-LN, [L, B, E]
    layer.train()
    xt = torch.from_numpy(X).transpose(0, 1).contiguous().requires_grad_(True)
    dyt = torch.from_numpy(DY).transpose(0, 1).contiguous()

    def torch_step():
        xt.grad = None
        layer.zero_grad(set_to_none=True)
        layer(xt).backward(dyt)

    def median_ms(fn):
        for _ in range(warmups):
            fn()
        ts = []
        for _ in range(runs):
            t0 = time.perf_counter(); fn(); ts.append(time.perf_counter() - t0)
        return round(statistics.median(ts) * 1e3, 2)

    try:
        from threadpoolctl import threadpool_info
        blas = sorted({f"{q.get('internal_api')} {q.get('num_threads')} threads" for q in threadpool_info()})
    except Exception:
        blas = []
    return {'workload': 'configs[0]: B=2 L=128 H=12 E=768 P=64 FF=3072 post-LN ReLU fp32 fwd+bwd, p=0.1',
            'numpy_oracle_ms': median_ms(numpy_step), 'torch_cpu_ms': median_ms(torch_step),
            'protocol': f'time.perf_counter, {warmups} warm-ups, median of {runs}',
            'logical_cpus': os.cpu_count(), 'torch_threads': torch.get_num_threads(),
            'omp_num_threads': os.environ.get('OMP_NUM_THREADS'), 'blas': blas}


def fused_op_rows(steps, warmup, only=None):
    """BASELINE configs[1] and the other memory-bound operators on their own, through the
    operator entry points of the C ABI (the units pytorch_module/benchmark.py times, whose
    shipped results are perf_softmax.txt, perf_bad.txt, perf_bsb.txt, perf_bdrln.txt):
    softmax forward (scale 1/8, p=0.1 seeded) and its backward on scores [H=16,B=8,J=512,K=512],
    every other operator at the shapes of B=8 L=512 E=1024 FF=4096.  Each operator cycles over
    enough buffer sets to exceed the 256 MiB memory-side cache; the launches of one round are
    recorded in a HIP graph and replayed, so that the HIP events around the replays time the
    GPU and not the Python caller.  GB/s = algorithmic bytes (each big tensor read once and
    written once) / time."""
    import torch
    from substation_amd.ops import Ops
    B, L, H, E = 8, 512, 16, 1024
    U = 4 * E
    o = Ops(B, L, H, E, activation='relu', seed=0x5EED + 2)
    g = torch.Generator(device='cuda').manual_seed(1002)
    bytes_of = {'HBJK': H * B * L * L * 2, 'BJI': B * L * E * 2, 'BJU': B * L * U * 2, 'QBJHP': 3 * B * L * E * 2}

    def randn(layout, std=1.0):
        t = o.empty(layout)
        t.normal_(0.0, std, generator=g)
        return t

    def vec(n, std=0.02, mean=0.0):
        return torch.empty(n, dtype=torch.float16, device='cuda').normal_(mean, std, generator=g)

    def keepmask(layout):
        return (torch.rand(o.empty(layout).shape, device='cuda', generator=g) >= 0.1).half()

    # operator -> (algorithmic tensors moved, their layout, make(): one buffer set, run(set))
    def softmax_set():
        return dict(beta=randn('HBJK'), alpha=o.empty('HBJK'), mask=o.empty('HBJK'), drop=o.empty('HBJK'))

    def bs_set():
        d = softmax_set()
        o.softmax(d['beta'], 'HBJK', d['alpha'], 'HBJK', d['mask'], 'HBJK', d['drop'], 'HBJK', scale=0.125, p=0.1)
        return dict(alpha=d['alpha'], mask=d['mask'], ddrop=randn('HBJK'), dbeta=d['beta'])

    def bdrln_set():
        return dict(inp=randn('BJI'), resid=randn('BJI'), lb=vec(E), s=vec(E, 0.1, 1.0), b=vec(E), mask=o.empty('BJI'),
                    diff=o.empty('BJI'), normed=o.empty('BJI'), out=o.empty('BJI'), istd=o.empty('BJ'))

    def blnrd_set():
        return dict(dout=randn('BJI'), istd=randn('BJ').abs_().add_(0.5), diff=randn('BJI'), mask=keepmask('BJI'),
                    a=o.empty('BJI'), b=o.empty('BJI'))

    def lnbwd_set(ext):
        d = dict(inp=randn('BJI'), s=vec(E, 0.1, 1.0), d1=randn('BJI'), istd=randn('BJ').abs_().add_(0.5),
                 diff=randn('BJI'), mask=keepmask('BJI'), g=o.empty('BJI'), a=o.empty('BJI'), b=o.empty('BJI'),
                 ds=vec(E), db=vec(E))
        if ext:
            d.update(d2=randn('BJI'), dl=randn('BJI'), dlb=vec(E), dob=vec(E))
        return d

    def run_lnbwd(d):
        if 'd2' in d:
            o.ln_backward(d['inp'], 'BJI', d['s'], d['d1'], 'BJI', d['istd'], 'BJ', d['diff'], 'BJI', d['mask'], 'BJI',
                          d['g'], 'BJI', d['a'], 'BJI', d['b'], 'BJI', d['ds'], d['db'], dout2=d['d2'], l_dout2='BJI',
                          dlinear=d['dl'], l_dlinear='BJI', dlinear_bias=d['dlb'], dout_bias=d['dob'])
        else:
            o.ln_backward(d['inp'], 'BJI', d['s'], d['d1'], 'BJI', d['istd'], 'BJ', d['diff'], 'BJI', d['mask'], 'BJI',
                          d['g'], 'BJI', d['a'], 'BJI', d['b'], 'BJI', d['ds'], d['db'])

    specs = [
        ('softmax', 4, 'HBJK', softmax_set,
         lambda d: o.softmax(d['beta'], 'HBJK', d['alpha'], 'HBJK', d['mask'], 'HBJK', d['drop'], 'HBJK',
                             scale=0.125, p=0.1)),
        ('bs', 4, 'HBJK', bs_set,
         lambda d: o.bs(d['alpha'], 'HBJK', d['mask'], 'HBJK', d['ddrop'], 'HBJK', d['dbeta'], 'HBJK', scale=0.125)),
        ('bdrln', 7, 'BJI', bdrln_set,
         lambda d: o.bdrln(d['inp'], 'BJI', d['resid'], 'BJI', d['lb'], d['s'], d['b'], d['inp'], 'BJI', d['mask'], 'BJI',
                           d['diff'], 'BJI', d['normed'], 'BJI', d['out'], 'BJI', d['istd'], 'BJ', p=0.1, site=1)),
        ('blnrd', 5, 'BJI', blnrd_set,
         lambda d: o.blnrd(d['dout'], 'BJI', d['istd'], 'BJ', d['diff'], 'BJI', d['mask'], 'BJI', d['a'], 'BJI',
                           d['b'], 'BJI')),
        ('bad', 4, 'BJU', lambda: dict(inp=randn('BJU'), bias=vec(U), lin=o.empty('BJU'), mask=o.empty('BJU'),
                                       out=o.empty('BJU')),
         lambda d: o.bad(d['inp'], 'BJU', d['bias'], d['lin'], 'BJU', d['mask'], 'BJU', d['out'], 'BJU', p=0.1, site=2)),
        ('bdrlb', 4, 'BJU', lambda: dict(dd=randn('BJU'), mask=keepmask('BJU'), lin=randn('BJU'), dl=o.empty('BJU'),
                                         db=vec(U)),
         lambda d: o.bdrlb(d['dd'], 'BJU', d['mask'], 'BJU', d['lin'], 'BJU', d['dl'], 'BJU', d['db'])),
        ('bsb', 3, 'BJI', lambda: dict(inp=randn('BJI'), s=vec(E, 0.1, 1.0), dout=randn('BJI'), din=o.empty('BJI'),
                                       ds=vec(E), db=vec(E)),
         lambda d: o.bsb(d['inp'], 'BJI', d['s'], d['dout'], 'BJI', d['din'], 'BJI', d['ds'], d['db'])),
        ('ebsb', 5, 'BJI', lambda: dict(inp=randn('BJI'), s=vec(E, 0.1, 1.0), d1=randn('BJI'), d2=randn('BJI'),
                                        dl=randn('BJI'), din=o.empty('BJI'), ds=vec(E), db=vec(E), dlb=vec(E)),
         lambda d: o.ebsb(d['inp'], 'BJI', d['s'], d['d1'], 'BJI', d['d2'], 'BJI', d['dl'], 'BJI', d['din'], 'BJI',
                          d['ds'], d['db'], d['dlb'])),
        ('bsb+blnrd', 7, 'BJI', lambda: lnbwd_set(False), run_lnbwd),
        ('ebsb+blnrd+baob', 9, 'BJI', lambda: lnbwd_set(True), run_lnbwd),
        ('baob', 1, 'BJI', lambda: dict(d=randn('BJI'), o=vec(E)), lambda d: o.baob(d['d'], 'BJI', d['o'])),
        ('aib', 2, 'QBJHP', lambda: dict(i=randn('QBJHP'), b=o.empty('QHP').normal_(0, 0.02, generator=g),
                                         o=o.empty('QBJHP')),
         lambda d: o.aib(d['i'], 'QBJHP', d['b'], 'QHP', d['o'], 'QBJHP')),
        ('baib', 1, 'QBJHP', lambda: dict(d=randn('QBJHP'), o=o.empty('QHP')),
         lambda d: o.baib(d['d'], 'QBJHP', d['o'], 'QHP')),
        ('bei', 3, 'BJI', lambda: dict(a=randn('BJI'), b=randn('BJI'), o=o.empty('BJI')),
         lambda d: o.bei(d['a'], 'BJI', d['b'], 'BJI', d['o'], 'BJI')),
    ]
    rows = []
    for name, ntens, layout, make, run in specs:
        if only is not None and name not in only:
            continue
        nbytes = ntens * bytes_of[layout]
        nsets = max(2, -(-(640 << 20) // nbytes))            # > 2.5 x the memory-side cache in rotation
        sets = [make() for _ in range(nsets)]
        for d in sets:                                        # warm-up; also allocates the handle's scratch
            run(d)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for d in sets:
                    run(d)
        torch.cuda.synchronize()
        for _ in range(max(1, warmup // 10)):
            graph.replay()
        reps = max(3, steps // 10)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e-3 / (reps * nsets)
        rows.append(dict(op=name, bound='hbm', us=round(t * 1e6, 2), achieved=round(nbytes / t / 1e9, 1),
                         unit='GB/s', frac=round(nbytes / t / HBM_PEAK, 4), bytes=nbytes, buffer_sets=nsets))
        del sets, graph
        torch.cuda.empty_cache()
    return rows


def bench_fused_ops(args):
    """`--config 2`: the line of the fused operators standing alone (fused_op_rows) beside the vendor's
    streaming kernels on tensors of the same sizes."""
    import torch
    rows = fused_op_rows(args.steps, args.warmup)
    # What the same box gives vendor streaming kernels of the same shapes (torch elementwise kernels, timed the
    # same way): a ceiling for 1 read + 1 write (copy), 2 reads + 1 write (add) and 1 write (fill) at the two
    # sizes the operators above have, 8 MiB and 64 MiB per tensor.
    stream = []
    for mib in (8, 64):
        n = mib << 19                                         # fp16 elements
        for kind, ntens in (('copy', 2), ('add', 3), ('fill', 1)):
            nbytes = ntens * n * 2
            nsets = max(2, -(-(640 << 20) // nbytes))
            sets = [[torch.empty(n, dtype=torch.float16, device='cuda').normal_() for _ in range(ntens)]
                    for _ in range(nsets)]

            def run(t, kind=kind):
                if kind == 'copy':
                    t[1].copy_(t[0])
                elif kind == 'add':
                    torch.add(t[0], t[1], out=t[2])
                else:
                    t[0].fill_(1.0)

            for t in sets:
                run(t)
            torch.cuda.synchronize()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                with torch.cuda.graph(graph, stream=side):
                    for t in sets:
                        run(t)
            torch.cuda.synchronize()
            graph.replay()
            reps = max(3, args.steps // 10)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            t_one = e0.elapsed_time(e1) * 1e-3 / (reps * nsets)
            stream.append(dict(kernel=f'torch {kind}, {mib} MiB per tensor', us=round(t_one * 1e6, 2),
                               gbps=round(nbytes / t_one / 1e9, 1), frac=round(nbytes / t_one / HBM_PEAK, 4)))
            del sets, graph
            torch.cuda.empty_cache()
    if args.per_op:
        for r in rows + stream:
            print(json.dumps(r), file=sys.stderr)
    sm = [r for r in rows if r['op'] in ('softmax', 'bs')]
    t_sm = sum(r['us'] for r in sm) * 1e-6
    b_sm = sum(r['bytes'] for r in sm)
    dom = max(sm, key=lambda r: r['us'])
    out = {
        'metric': 'fused-op HBM GB/s vs peak: softmax forward + backward alone, [H=16,B=8,J=512,K=512] fp16',
        'value': round(b_sm / t_sm / 1e9, 1), 'unit': 'GB/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': round(t_sm * 1e3, 4), 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'fp16', 'data': 'synthetic',
        'config': {'workload': 'configs[1]: softmax (scale 1/8, dropout p=0.1 seeded) + softmax backward on scores '
                               '[16,8,512,512]; the other fused operators at B=8 L=512 E=1024 FF=4096, each alone'},
        'roofline': {'kernel': dom['op'], 'bound': 'hbm', 'achieved': dom['achieved'], 'peak': HBM_PEAK / 1e9,
                     'unit': 'GB/s', 'frac': dom['frac'], 'traffic': None, 'launch_us': dom['us']},
        'reference_published_us': {'softmax (1 read + 1 write, no dropout outputs)': 187.97, 'bad (p=0)': 91.45,
                                   'bsb': 72.97, 'bdrln (p=0)': 51.53,
                                   'source': 'pytorch_module/perf_softmax.txt, perf_bad.txt, perf_bsb.txt, '
                                             'perf_bdrln.txt (GPU not stated)'},
        'ops': [{k: r[k] for k in ('op', 'us', 'achieved', 'unit', 'frac', 'bytes', 'buffer_sets')} for r in rows],
        'stream_reference': stream,
    }
    print(json.dumps(out))


def bench_fetch_probe(args):
    """What 256 CUs draw from the L2s and from beyond them (sub_probe_fetch): a table on stdout, one line
    per working set and load form.  The contraction kernels' operand fetch is priced against these rates."""
    import ctypes
    import torch
    from substation_amd import _lib
    lib = _lib.load()
    cap = 1 << 30
    buf = torch.empty(cap, dtype=torch.uint8, device='cuda').fill_(1)
    torch.cuda.synchronize()
    us, mhz = ctypes.c_float(), ctypes.c_float()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    print(f'{"working set":>12s}  {"load form":20s} {"workgroups":>10s} {"us":>8s} {"TB/s":>6s} {"GB/s per CU":>11s} {"MHz":>5s} {"bytes/clk per CU":>16s}')
    rows = [(ws, form, 256) for ws in (1 << 20, 2 << 20, 8 << 20, 32 << 20, 128 << 20, 1 << 30) for form in (1, 0)]
    rows += [(2 << 20, 1, 64), (2 << 20, 1, 8)]
    # copy and fill of tensor-sized regions, every chunk once, at several occupancies (workgroups x iterations = chunks)
    rows += [(ws, form, wgs) for ws in (8 << 20, 64 << 20, 512 << 20) for form in (2, 3) for wgs in (128, 256, 1024)
             if wgs <= ws // 65536 and (wgs == 128) == (ws == 8 << 20)]
    names = {0: '128-bit to registers', 1: 'asynchronous to LDS', 2: 'copy (read + write)', 3: 'fill (write)'}
    for ws, form, wgs in rows:
        iters = 64 if form < 2 else max(1, ws // 65536 // wgs)
        _lib.check(lib.sub_probe_fetch(ctypes.c_void_p(buf.data_ptr()), ws, form, iters, wgs, stream, ctypes.byref(us),
                                       ctypes.byref(mhz)), 'sub_probe_fetch')
        nbytes = 65536.0 * iters * wgs * (2 if form == 2 else 1)
        print(f'{ws / 2**20:8.0f} MiB  {names[form]:20s} {wgs:10d} {us.value:8.1f} '
              f'{nbytes / us.value / 1e6:6.2f} {nbytes / us.value / 1e3 / min(wgs, 256):11.1f} {mhz.value:5.0f} '
              f'{nbytes / min(wgs, 256) / (us.value * mhz.value):16.1f}')


def bench_decoder(cfg, args):
    """Forward + backward of substation_amd.DecoderLayer (substation/transformer.py:288-441), not the headline
    metric: one JSON line of its own."""
    import torch
    from substation_amd import DecoderLayer
    B, L, H, E = cfg['B'], cfg['L'], cfg['H'], cfg['E']
    layer = DecoderLayer(B, L, L, H, E, 0.1, 0.1, 0.1, 0.1, activation=cfg.get('act', 'relu'), seed=0x5EED,
                         intermediate_size=cfg.get('U')).cuda()
    g = torch.Generator().manual_seed(1000 + args.config)
    x = torch.randn(B, L, E, generator=g).half().cuda().requires_grad_(True)
    enc_out = torch.randn(B, L, E, generator=g).half().cuda().requires_grad_(True)
    dy = torch.randn(B, L, E, generator=g).half().cuda()
    params = list(layer.parameters())

    def step():
        x.grad = None; enc_out.grad = None
        for q in params:
            q.grad = None
        layer(x, enc_out).backward(dy)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    print(json.dumps({'metric': 'fwd+bwd ms/decoder layer with encoder-decoder attention', 'value': round(ms, 4),
                      'unit': 'ms', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
                      'ms_per_step': round(ms, 4), 'higher_is_better': False, 'dtype': 'fp16', 'data': 'synthetic',
                      'vs_baseline': None,
                      'config': {'workload': f'decoder layer B={B} target=source={L} H={H} E={E} causal, 4 dropouts p=0.1'}}))


def make_step(enc, X, DY):
    """One training step of the layer: forward, then backward from DY (run_encoder.py:361-368)."""
    params = list(enc.parameters())

    def step():
        X.grad = None
        for q in params:       # as optimizer.zero_grad(set_to_none=True): no accumulate kernels
            q.grad = None
        Y = enc(X)
        Y.backward(DY)
    return step


def lead_steps(ms_per_step):
    """How many steps to issue in front of a measured one so that the host is a whole step ahead of
    the GPU when the measured step begins (the host issues a step in roughly half the time the GPU
    takes for it; fewer for long steps)."""
    return max(3, min(10, int(6.0 / max(ms_per_step, 0.05)) + 1))


def preheat(step, ms_per_step, ms=150.0):
    """Runs the step itself for about `ms` milliseconds.  After an idle period of a few tens of
    milliseconds the device is slow for the next ten to twenty milliseconds of work (0.55 ms per
    step falling to 0.49 at the bench workload, measured; a spin kernel does not prevent it, real
    memory traffic does): whatever is to be compared with steady-state figures -- the reference's are
    medians of 1000 iterations after 100 warm-ups, pytorch_module/run_encoder.py:34-38 -- is measured
    behind this."""
    import torch
    n = int(ms / max(ms_per_step, 0.05)) + 1
    for _ in range(n):
        step()
    torch.cuda.synchronize()
    return n


def timed_steps(step, steps, warmup):
    """The timed region: `warmup` untimed steps, then `steps` steps between two synchronisations on
    the host clock; ms per step."""
    import torch
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def gpu_step_us(step, n, lead):
    """GPU time of one step in microseconds: n steps behind `lead` steps of the same workload (which
    keep the device at its working clocks and give the host its lead, so that the figure does not
    depend on how fast this host issues launches), from an event in front of the first to one
    behind the last."""
    import torch
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(lead):
        step()
    e0.record()
    for _ in range(n):
        step()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / n


def pass_times(enc, X, DY, n, lead):
    """Forward and backward pass timed apart, as pytorch_module/run_encoder.py:359-383 does: an event
    before the forward call, one between the passes, one after the backward call, n steps in a row
    behind `lead` untimed ones; median, min, max and standard deviation of each pass in ms (the
    three events of a step cost a few microseconds, which stay in the figures)."""
    import torch
    params = list(enc.parameters())
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(n)]

    def one(a=None, b=None, c=None):
        X.grad = None
        for q in params:
            q.grad = None
        if a is not None:
            a.record()
        Y = enc(X)
        if b is not None:
            b.record()
        Y.backward(DY)
        if c is not None:
            c.record()
    for _ in range(lead):
        one()
    for a, b, c in evs:
        one(a, b, c)
    torch.cuda.synchronize()
    done = [(a.elapsed_time(b), b.elapsed_time(c)) for a, b, c in evs]
    out = {}
    for name, ts in (('forward', [d[0] for d in done]), ('backward', [d[1] for d in done])):
        out[name] = {'median_ms': round(statistics.median(ts), 4), 'min_ms': round(min(ts), 4),
                     'max_ms': round(max(ts), 4), 'stdev_ms': round(statistics.pstdev(ts), 4)}
    out['steps'] = len(done)
    return out


def other_workloads(args):
    """The BASELINE workloads the headline figure does not cover, each for a fraction of a second of GPU
    time: configs[3] and configs[4] as ms per layer (the headline's protocol -- warm-ups, then steps
    between two synchronisations on the host clock, behind the same preheating -- and the GPU's own time per
    step), configs[1] as the fused operators standing alone on buffers larger than the memory-side cache."""
    import torch
    out = {}
    for cid, steps, warmup in ((4, 20, 5), (5, 6, 2)):
        cfg = dict(CONFIGS[cid])
        enc, X, DY = make_encoder(cfg, args.layouts)
        step = make_step(enc, X, DY)
        step()                                   # (allocations)
        torch.cuda.synchronize()
        pre = preheat(step, 1.3 if cid == 4 else 11.0)           # building the layer left the device idle
        ms = timed_steps(step, steps, warmup)
        gpu_ms = gpu_step_us(step, min(steps, 10), lead_steps(ms)) * 1e-3
        U, P = 4 * cfg['E'], cfg['E'] // cfg['H']
        flops = 3 * (2 * cfg['B'] * cfg['L'] * (4 * cfg['E'] ** 2 + 2 * cfg['E'] * U)
                     + 4 * cfg['B'] * cfg['H'] * cfg['L'] ** 2 * P)
        out['configs[%d]' % (cid - 1)] = {'workload': cfg['name'], 'ms_per_layer': round(ms, 4),
                                          'gpu_ms_per_layer': round(gpu_ms, 4), 'steps': steps, 'warmup': warmup,
                                          'preheat_steps': pre,
                                          'tflops': round(flops / (gpu_ms * 1e-3) / 1e12, 1),
                                          'frac_of_mfma_peak': round(flops / (gpu_ms * 1e-3) / MFMA_PEAK_F16, 4)}
        del enc, X, DY, step
        torch.cuda.empty_cache()
    rows = fused_op_rows(30, 10, only=('softmax', 'bs', 'bad', 'bdrln'))
    out['configs[1]'] = {'workload': 'softmax (scale 1/8, dropout p=0.1 seeded) and its backward on scores [16,8,512,512], '
                                     'bad and bdrln at B=8 L=512 E=1024 FF=4096, each operator alone, fp16 masks and every '
                                     'output written (the reference operators\' tensors)',
                         'ops': [{k: r[k] for k in ('op', 'us', 'achieved', 'unit', 'frac', 'bytes')} for r in rows]}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=200)
    ap.add_argument('--warmup', type=int, default=30)
    ap.add_argument('--config', type=int, default=3, choices=[2] + sorted(CONFIGS))
    ap.add_argument('--layouts', default='mi355x', choices=['mi355x', 'ref'])
    ap.add_argument('--profile-steps', type=int, default=20)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-other-workloads', action='store_true',
                    help='leave out the short runs of BASELINE configs[1], [3] and [4] that the default line carries')
    ap.add_argument('--per-op', action='store_true', help='print the per-operator table to stderr')
    ap.add_argument('--option', action='append', default=[], metavar='ID=VALUE',
                    help='library option to set (sub_set_option), e.g. 2=0 runs the LayerNorm backward '
                         'as separate launches')
    ap.add_argument('--copy-calibration', action='store_true',
                    help='also run 5 device copies of 256 MiB (known traffic) for scaling rocprofv3 '
                         'FETCH_SIZE / WRITE_SIZE readings')
    ap.add_argument('--preheat-ms', type=float, default=None,
                    help='milliseconds of the workload itself run before the timed region is repeated for `value` '
                         '(default 150; 0: `value` is the cold-start figure; with --profile-steps 0 the default is 0 and '
                         'the one timed region runs behind the preheating)')
    ap.add_argument('--fetch-probe', action='store_true',
                    help='measure what the CUs draw from the L2s and from beyond them (a table, no JSON line)')
    ap.add_argument('--activation', choices=['relu', 'gelu'], default=None,
                    help="the feed-forward activation, instead of the configuration's own (then named in config.workload)")
    ap.add_argument('--decoder', action='store_true',
                    help='time the decoder layer with encoder-decoder attention (both lengths = the '
                         "configuration's L, causal self-attention) instead of the encoder layer; prints its own line")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py: this build runs the encoder layer on ONE GPU only (no collectives exist on '
              'this path); run with --gpus 1', file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print('bench.py: no GPU visible', file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    if args.fetch_probe:
        bench_fetch_probe(args)
        return
    if args.config == 2:
        bench_fused_ops(args)
        return
    cfg = dict(CONFIGS[args.config])
    if args.activation and args.activation != cfg['act']:
        cfg['act'] = args.activation
        cfg['name'] += ' [activation: %s]' % args.activation
    if args.decoder:
        bench_decoder(cfg, args)
        return
    enc, X, DY = make_encoder(cfg, args.layouts)
    for item in args.option:
        k, v = item.split('=')
        enc._handle.set_option(int(k), int(v))
    step = make_step(enc, X, DY)

    # The timed region twice: as the process finds the device (idle since the module was built), and again
    # behind 150 ms of the same steps.  The second is `value`: the steady state, which is what the reference's
    # published figures are; the first is kept beside it as cold_start_ms_per_step.
    # (Timing-only runs, --profile-steps 0, are what the profiler is pointed at: one timed region, behind the
    # preheating when --preheat-ms is given.)
    timing_only = args.profile_steps <= 0
    preheat_ms = args.preheat_ms if args.preheat_ms is not None else (0.0 if timing_only else 150.0)
    preheat_steps = 0
    if timing_only:
        if preheat_ms > 0:
            step()
            torch.cuda.synchronize()
            preheat_steps = preheat(step, 0.55 * cfg['B'] * cfg['L'] / 4096 * (cfg['E'] / 1024) ** 2, preheat_ms)
        cold_ms = ms_per_step = timed_steps(step, args.steps, args.warmup)
    else:
        cold_ms = ms_per_step = timed_steps(step, args.steps, args.warmup)
        if preheat_ms > 0:
            preheat_steps = preheat(step, cold_ms, preheat_ms)
            ms_per_step = timed_steps(step, args.steps, args.warmup)

    if args.copy_calibration:
        a = torch.empty(128 << 20, dtype=torch.float16, device='cuda').normal_()
        b = torch.empty_like(a)
        for _ in range(5):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b

    if args.profile_steps <= 0:        # timing only
        print(json.dumps({'metric': 'fwd+bwd ms/layer', 'value': round(ms_per_step, 4), 'unit': 'ms',
                          'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'preheat_steps': preheat_steps,
                          'ms_per_step': round(ms_per_step, 4), 'higher_is_better': False}))
        return

    # Everything below is timed on the GPU's own clock (HIP events on the launch stream) behind a few steps
    # of the same workload, so that the host has issued the launches before they run and the device is at its
    # working clocks: a figure does not depend on how fast this host issues them.
    lead = lead_steps(ms_per_step)
    # Forward and backward pass apart, an event between them (pytorch_module/run_encoder.py:359-383).
    passes = pass_times(enc, X, DY, max(10, min(args.steps, 50)), lead)
    # The cost of the library's per-launch events, calibrated directly: the same steps back to back with
    # and without them, in turns; the difference per launch is taken off every entry below.
    n_cal = 10
    plain, inst = [], []
    for _ in range(3):
        plain.append(gpu_step_us(step, n_cal, lead))
        enc._handle.profile_enable(True)
        inst.append(gpu_step_us(step, n_cal, lead))
        enc._handle.profile_enable(False)
    gpu_us_per_step = statistics.median(plain)
    # Per-launch durations: an event in front of every launch and one at the end of each pass, a launch
    # lasting from its event to the next; the launches are the timed region's.
    enc._handle.profile_enable(True)
    per_op = {}
    for _ in range(args.profile_steps):
        for _ in range(lead + 1):          # the last one is read
            step()
        for n, ms in enc.profile():
            per_op.setdefault(n, []).append(ms)
    # The shader clock the GPU held during each launch (a one-lane kernel in front of every launch samples the
    # clock counters; a pass of its own, durations are not taken from it): the matrix-core peak scales with it.
    enc._handle.profile_enable(2)
    clocks = {}
    for _ in range(min(5, args.profile_steps)):
        for _ in range(lead + 1):
            step()
        for n, mhz in enc._handle.profile_read_clocks():
            clocks.setdefault(n, []).append(mhz)
    enc._handle.profile_enable(False)
    staged = staged_elements(enc.layouts, cfg['B'], cfg['L'], cfg['H'], cfg['E']) if '11=0' not in args.option else (0, 0)
    work = algorithmic_work(cfg['B'], cfg['L'], cfg['H'], cfg['E'],
                            relu_from_output=cfg['act'] == 'relu' and '6=0' not in args.option,
                            packed_masks='9=0' not in args.option and cfg['E'] % 8 == 0,
                            skip_unread='10=0' not in args.option, staged=staged)
    # Memory-bound launches: `achieved` and `frac` are the bytes the launch moves (each big tensor it reads
    # or writes once, the residual dropout masks as bits, outputs nothing reads not written) per second; what
    # the reference's operators would have moved for the same result (masks as fp16 tensors, every named
    # output written) is reported beside it as effective_gbps_ref_bytes.
    work_ref = algorithmic_work(cfg['B'], cfg['L'], cfg['H'], cfg['E'],
                                relu_from_output=cfg['act'] == 'relu' and '6=0' not in args.option,
                                packed_masks=False, skip_unread=False, staged=staged)
    raw_us = {n: statistics.mean(ts) * 1e3 for n, ts in per_op.items()}
    event_us = (statistics.median(inst) - gpu_us_per_step) / max(1, len(raw_us))
    ops = []
    for n in per_op:
        t = max(raw_us[n] - event_us, 0.5) * 1e-6
        kind = work[n]
        if kind[0] == 'hbm':
            ref_bytes = work_ref[n][1]
            ops.append(dict(op=n, bound='hbm', us=round(t * 1e6, 2), achieved=round(kind[1] / t / 1e9, 1),
                            peak=HBM_PEAK / 1e9, unit='GB/s', frac=round(kind[1] / t / HBM_PEAK, 4),
                            bytes=kind[1], ref_bytes=ref_bytes,
                            effective_gbps_ref_bytes=round(ref_bytes / t / 1e9, 1)))
            if clocks.get(n):
                ops[-1]['mhz'] = round(statistics.median(clocks[n]))
        else:
            o = dict(op=n, bound='mfma', us=round(t * 1e6, 2), achieved=round(kind[1] / t / 1e12, 1),
                     peak=MFMA_PEAK_F16 / 1e12, unit='TFLOP/s', frac=round(kind[1] / t / MFMA_PEAK_F16, 4),
                     flops=kind[1], flops_algorithmic=kind[3] if len(kind) > 3 else kind[1],
                     hbm_gbps=round(kind[2] / t / 1e9, 1))
            if clocks.get(n):
                # fraction of what the matrix cores could do at the clock they ran at (peak is quoted at 2400 MHz)
                o['mhz'] = round(statistics.median(clocks[n]))
                o['frac_at_clock'] = round(kind[1] / t / (MFMA_PEAK_F16 * o['mhz'] / PEAK_MHZ), 4)
            if len(kind) > 3:      # attention: the scores are formed again in the backward launches
                o['achieved_algorithmic'] = round(kind[3] / t / 1e12, 1)
                o['frac_algorithmic'] = round(kind[3] / t / MFMA_PEAK_F16, 4)
            ops.append(o)
    ops.sort(key=lambda o: -o['us'])
    dom = ops[0]
    total_us = sum(o['us'] for o in ops)
    fused = [o for o in ops if o['bound'] == 'hbm']
    gemms = [o for o in ops if o['bound'] == 'mfma']
    fused_s = sum(o['us'] for o in fused) * 1e-6
    gemm_s = sum(o['us'] for o in gemms) * 1e-6
    if args.per_op:
        for o in ops:
            print(json.dumps(o), file=sys.stderr)

    # the headline workload as configured: another activation is another workload (no published figure, no tracked traffic)
    headline = args.config == 3 and cfg['act'] == CONFIGS[3]['act']
    out = {
        # `value` is the first half of the metric (ms/layer); the second half is in `fused_ops` and `ops`
        'metric': ('fwd+bwd ms/layer BERT-large B8 L512 fp16; fused-op HBM GB/s vs peak' if headline
                   else 'fwd+bwd ms/layer'),
        'value': round(ms_per_step, 4), 'unit': 'ms', 'n_gpus': 1, 'steps': args.steps,
        'warmup': args.warmup, 'ms_per_step': round(ms_per_step, 4), 'higher_is_better': False,
        'scaling': 'weak', 'vs_baseline': round(ms_per_step / V100_MS, 4) if headline else None,
        # the same timed region as the process found the device, before `preheat_steps` steps of the workload
        'cold_start_ms_per_step': round(cold_ms, 4), 'preheat_steps': preheat_steps,
        'dtype': 'fp16', 'data': 'synthetic',
        'config': {'workload': cfg['name'], 'layouts': args.layouts,
                   'baseline': 'reference README.md:23: 6.71 ms on V100-SXM2 (other hardware)'},
        'roofline': {
            'kernel': dom['op'], 'bound': dom['bound'], 'achieved': dom['achieved'], 'peak': dom['peak'],
            'unit': dom['unit'], 'frac': dom['frac'],
            'traffic': (measured_traffic().get(dom['op']) if headline and args.layouts == 'mi355x'
                        and not args.option else None),
            'launch_us': dom['us'], 'launches_per_step': 1,
        },
        # GPU time of a step without and with the per-launch events, steps back to back;
        # their difference per launch is what was taken off every entry of `ops`
        'gpu_us_per_step': round(gpu_us_per_step, 1), 'gpu_us_per_step_with_events': round(statistics.median(inst), 1),
        'op_time_us': round(total_us, 1), 'event_us_per_launch': round(event_us, 2),
        'passes': passes,
        'fused_ops': {'us': round(fused_s * 1e6, 1),
                      'gbps': round(sum(o['bytes'] for o in fused) / fused_s / 1e9, 1),
                      'frac_of_hbm_peak': round(sum(o['bytes'] for o in fused) / fused_s / HBM_PEAK, 4),
                      'bytes': 'what the launches move: each big tensor once, residual dropout masks as bits',
                      'effective_gbps_ref_bytes': round(sum(o['ref_bytes'] for o in fused) / fused_s / 1e9, 1)},
        # flops: the 18 products of the layer (attention without the scores formed a second time in the
        # backward launches); executed_tflops counts those as well
        'contractions': {'us': round(gemm_s * 1e6, 1),
                         'tflops': round(sum(o['flops_algorithmic'] for o in gemms) / gemm_s / 1e12, 1),
                         'frac_of_mfma_peak': round(sum(o['flops_algorithmic'] for o in gemms) / gemm_s / MFMA_PEAK_F16, 4),
                         'executed_tflops': round(sum(o['flops'] for o in gemms) / gemm_s / 1e12, 1)},
        'ops': [{k: o[k] for k in ('op', 'bound', 'us', 'achieved', 'unit', 'frac', 'effective_gbps_ref_bytes',
                                   'achieved_algorithmic', 'frac_algorithmic', 'mhz', 'frac_at_clock') if k in o}
                for o in ops],
    }
    del enc, X, DY, step
    torch.cuda.empty_cache()
    if headline and args.layouts == 'mi355x' and not args.option and not args.no_other_workloads:
        out['other_workloads'] = other_workloads(args)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(out))


if __name__ == '__main__':
    main()
