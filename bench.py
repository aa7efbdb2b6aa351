"""Benchmark of the fused encoder layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 3|4|5] [--layouts mi355x|ref]

A step is one forward + one backward pass of a single encoder layer over one
batch of synthetic input (the protocol of pytorch_module/run_encoder.py:345-383).
The default workload is BERT-large B=8 L=512 H=16 E=1024 fp16 with the four
dropouts at p=0.1.  Prints ONE JSON line: ms per layer, the per-operator
roofline measured live with HIP events on the launch stream, and the CPU
baseline (the NumPy oracle on the reference's own CPU-sized case).
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

# HBM-side bytes per launch at the default workload and layouts: rocprofv3 FETCH_SIZE (x2.000) +
# WRITE_SIZE (x1.000), scale factors from a 256 MiB device copy; see
# profiles/encoder_layer_b8_l512_hbm_traffic.txt for the commands and the table.
MEASURED_TRAFFIC_CFG3 = {
    'QKV-fused': 91452057, 'attention': 38114912, 'out': 33775005, 'bdrln1': 59014043,
    'lin1+bad': 87734212, 'lin2': 109264774, 'bdrln2': 59016749, 'bsb+blnrd1': 61022384,
    'dXlin2+bdrlb': 118260844, 'dWlin2': 109269143, 'dXlin1+dWlin1': 298726901, 'ebsb+blnrd2+baob': 79940065,
    'dXout': 33752717, 'attention-bwd-dQ': 55316836, 'attention-bwd-dKdV': 55518567, 'dXQKV-fused+dWQKV-fused+dWout': 373479999,
}

GEMM_OPS = ('QKV-fused', 'QKT', 'gamma', 'out', 'lin1', 'lin2', 'dXlin2', 'dWlin2', 'dXlin1', 'dWlin1',
            'dWout', 'dXout', 'dX1gamma', 'dX2gamma', 'dX1QKT', 'dX2QKT', 'dXQKV-fused', 'dWQKV-fused')


def algorithmic_work(B, L, H, E, relu_from_output=True):
    """Per operator: ('hbm', bytes) or ('mfma', flops, bytes).  Bytes = each big
    tensor read once + written once in fp16; flops = 2*batch*M*N*K.
    relu_from_output: the ReLU layer as it runs by default -- bad writes only its
    output (one [B,J,U] tensor in, one out) and bdrlb reads the gate off that output
    (two in, one out); otherwise both move four."""
    U, P = 4 * E, E // H
    bji, bju, hbjk, q = B * L * E, B * L * U, H * B * L * L, 3 * B * L * E
    w = {
        'aib': ('hbm', 2 * q * 2), 'softmax': ('hbm', 4 * hbjk * 2), 'bs': ('hbm', 4 * hbjk * 2),
        'bdrln1': ('hbm', 7 * bji * 2), 'bdrln2': ('hbm', 7 * bji * 2),
        'blnrd1': ('hbm', 5 * bji * 2), 'blnrd2': ('hbm', 5 * bji * 2),
        'bsb': ('hbm', 3 * bji * 2), 'ebsb': ('hbm', 5 * bji * 2), 'baob': ('hbm', bji * 2),
        'bei': ('hbm', 3 * bji * 2), 'bad': ('hbm', (2 if relu_from_output else 4) * bju * 2),
        'bdrlb': ('hbm', (3 if relu_from_output else 4) * bju * 2),
        'baib': ('hbm', q * 2),
        # single-launch forms: the scaled gradient is written but not read back
        # (bsb + blnrd1 - one [B,J,I] read; ebsb + blnrd2 + baob - two reads)
        'bsb+blnrd1': ('hbm', 7 * bji * 2), 'ebsb+blnrd2+baob': ('hbm', 9 * bji * 2),
        # scores formed in place: the score tensor itself is neither written nor read
        # (QKT + softmax: Q, K in, three score-sized tensors out; dX1gamma + bs: dO, V
        # and two score-sized tensors in, one out)
        'QKT+softmax': ('hbm', (3 * hbjk + 2 * bji) * 2), 'dX1gamma+bs': ('hbm', (3 * hbjk + 2 * bji) * 2),
    }
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
    w['attention'] = ('mfma', 2 * attn[0], 2 * 4 * bji + hbjk // 8)
    w['attention-bwd-dQ'] = ('mfma', 3 * attn[0], 2 * 6 * bji + hbjk // 8)
    w['attention-bwd-dKdV'] = ('mfma', 4 * attn[0], 2 * 6 * bji + hbjk // 8)
    # two products in one launch
    w['dXlin1+dWlin1'] = ('mfma', 2 * ffn[0], 2 * ffn[1])
    w['dXQKV-fused+dWQKV-fused'] = ('mfma', 2 * proj[0], 2 * proj[1])
    w['dXout+dWout'] = ('mfma', 2 * outp[0], 2 * outp[1])
    # the last launch of the backward pass with dWout's tiles in the places it leaves free
    w['dXQKV-fused+dWQKV-fused+dWout'] = ('mfma', 2 * proj[0] + outp[0], 2 * proj[1] + outp[1])
    # lin1 with bias, ReLU and dropout in its epilogue: the product's flops, SB1 and LINW1 in, DROP2 out
    w['lin1+bad'] = ('mfma',) + ffn
    w['dXlin2+bdrlb'] = ('mfma', ffn[0], ffn[1] + 2 * tok * U)      # the product's bytes plus the gate (DROP2) read
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
    }


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=200)
    ap.add_argument('--warmup', type=int, default=30)
    ap.add_argument('--config', type=int, default=3, choices=sorted(CONFIGS))
    ap.add_argument('--layouts', default='mi355x', choices=['mi355x', 'ref'])
    ap.add_argument('--profile-steps', type=int, default=20)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--per-op', action='store_true', help='print the per-operator table to stderr')
    ap.add_argument('--option', action='append', default=[], metavar='ID=VALUE',
                    help='library option to set (sub_set_option), e.g. 2=0 runs the LayerNorm backward '
                         'as separate launches')
    ap.add_argument('--copy-calibration', action='store_true',
                    help='also run 5 device copies of 256 MiB (known traffic) for scaling rocprofv3 '
                         'FETCH_SIZE / WRITE_SIZE readings')
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
    cfg = CONFIGS[args.config]
    if args.decoder:
        bench_decoder(cfg, args)
        return
    enc, X, DY = make_encoder(cfg, args.layouts)
    for item in args.option:
        k, v = item.split('=')
        enc._handle.set_option(int(k), int(v))

    params = list(enc.parameters())

    def step():
        X.grad = None
        for q in params:       # as optimizer.zero_grad(set_to_none=True): no accumulate kernels
            q.grad = None
        Y = enc(X)
        Y.backward(DY)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    if args.copy_calibration:
        a = torch.empty(128 << 20, dtype=torch.float16, device='cuda').normal_()
        b = torch.empty_like(a)
        for _ in range(5):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b

    # Per-operator durations: HIP events recorded by the library around every
    # launch, on the stream the kernels run on.
    enc._handle.profile_enable(True)
    per_op = {}
    for _ in range(args.profile_steps):
        X.grad = None
        for q in params:
            q.grad = None
        Y = enc(X)
        for n, ms in enc.profile():
            per_op.setdefault(n, []).append(ms)
        Y.backward(DY)
        for n, ms in enc.profile():
            per_op.setdefault(n, []).append(ms)
    enc._handle.profile_enable(False)
    work = algorithmic_work(cfg['B'], cfg['L'], cfg['H'], cfg['E'],
                            relu_from_output=cfg['act'] == 'relu' and '6=0' not in args.option)
    ops = []
    for n, ts in per_op.items():
        t = statistics.mean(ts) * 1e-3
        kind = work[n]
        if kind[0] == 'hbm':
            ops.append(dict(op=n, bound='hbm', us=round(t * 1e6, 2), achieved=round(kind[1] / t / 1e9, 1),
                            peak=HBM_PEAK / 1e9, unit='GB/s', frac=round(kind[1] / t / HBM_PEAK, 4),
                            bytes=kind[1]))
        else:
            ops.append(dict(op=n, bound='mfma', us=round(t * 1e6, 2), achieved=round(kind[1] / t / 1e12, 1),
                            peak=MFMA_PEAK_F16 / 1e12, unit='TFLOP/s', frac=round(kind[1] / t / MFMA_PEAK_F16, 4),
                            flops=kind[1], hbm_gbps=round(kind[2] / t / 1e9, 1)))
    ops.sort(key=lambda o: -o['us'])
    if not ops:        # --profile-steps 0: timing only
        print(json.dumps({'metric': 'fwd+bwd ms/layer', 'value': round(ms_per_step, 4), 'unit': 'ms',
                          'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
                          'ms_per_step': round(ms_per_step, 4), 'higher_is_better': False}))
        return
    dom = ops[0]
    total_us = sum(o['us'] for o in ops)
    fused = [o for o in ops if o['bound'] == 'hbm']
    gemms = [o for o in ops if o['bound'] == 'mfma']
    if args.per_op:
        for o in ops:
            print(json.dumps(o), file=sys.stderr)

    out = {
        # `value` is the first half of the metric (ms/layer); the second half is in `fused_ops` and `ops`
        'metric': ('fwd+bwd ms/layer BERT-large B8 L512 fp16; fused-op HBM GB/s vs peak' if args.config == 3
                   else 'fwd+bwd ms/layer'),
        'value': round(ms_per_step, 4), 'unit': 'ms', 'n_gpus': 1, 'steps': args.steps,
        'warmup': args.warmup, 'ms_per_step': round(ms_per_step, 4), 'higher_is_better': False,
        'scaling': 'weak', 'vs_baseline': round(ms_per_step / V100_MS, 4) if args.config == 3 else None,
        'dtype': 'fp16', 'data': 'synthetic',
        'config': {'workload': cfg['name'], 'layouts': args.layouts,
                   'baseline': 'reference README.md:23: 6.71 ms on V100-SXM2 (other hardware)'},
        'roofline': {
            'kernel': dom['op'], 'bound': dom['bound'], 'achieved': dom['achieved'], 'peak': dom['peak'],
            'unit': dom['unit'], 'frac': dom['frac'],
            'traffic': (MEASURED_TRAFFIC_CFG3.get(dom['op']) if args.config == 3 and args.layouts == 'mi355x'
                        else None),
            'launch_us': dom['us'], 'launches_per_step': 1,
        },
        'op_time_us': round(total_us, 1),
        'fused_ops': {'us': round(sum(o['us'] for o in fused), 1),
                      'gbps': round(sum(o['bytes'] for o in fused) / (sum(o['us'] for o in fused) * 1e-6) / 1e9, 1),
                      'frac_of_hbm_peak': round(sum(o['bytes'] for o in fused) / (sum(o['us'] for o in fused) * 1e-6) / HBM_PEAK, 4)},
        'contractions': {'us': round(sum(o['us'] for o in gemms), 1),
                         'tflops': round(sum(o['flops'] for o in gemms) / (sum(o['us'] for o in gemms) * 1e-6) / 1e12, 1),
                         'frac_of_mfma_peak': round(sum(o['flops'] for o in gemms) / (sum(o['us'] for o in gemms) * 1e-6) / MFMA_PEAK_F16, 4)},
        'ops': [{k: o[k] for k in ('op', 'bound', 'us', 'achieved', 'unit', 'frac')} for o in ops],
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(out))


if __name__ == '__main__':
    main()
