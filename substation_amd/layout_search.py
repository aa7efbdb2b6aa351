"""Layout selection for the encoder layer from timings measured on the GPU.

What the reference does in three offline stages -- time every operator under
every layout with one nvcc build each (pytorch_module/benchmark.py:178-302,
1362-1472; tc_profiling/einsum_perms.py:352-470), load the tables
(config_selection/ops.py), and pick one layout per tensor that minimises the
summed operator times under the shared-tensor constraints
(config_selection/optimize.py:13-493, shortest path over a chain of operators)
-- happens here in one process.  The kernels take strides at run time, so a
candidate configuration is only a new handle: the whole layer is run under it
with per-operator timing on and the measured times are entered in the same
kind of table (operator x layouts of its tensors -> seconds, minimum over
measurements).  The minimisation is a coordinate descent over that table with
four kinds of moves (all same-shaped tensors of the layer; those together with
the weights of the operators that touch them, every combination of their layouts
as one coordinate; all same-shaped tensors of one operator; one tensor), measuring
only configurations whose operators are not all in the table yet.  The second
kind is what lets the descent leave the family of layouts it was started in
(feature-major activations, as in the reference's shipped configurations, against
token-major ones): the fused paths switch on for a whole group of tensors or
not at all.  Configurations that would send a
contraction to the scalar fallback kernel are discarded without being run.

Output: a layouts pickle in the schema of config_selection/optimize.py:443-493
(``save_configuration``) and, optionally, one line per table entry in the
format of pytorch_module/benchmark.py:1437-1441 (``k = v ... time = X s``).

    python -m substation_amd.layout_search --batch 8 --seq 512 --heads 16 \\
        --embed 1024 --out layouts-mi355x-bert-b8-l512-h16-e1024.pickle
"""
import argparse
import ctypes
import itertools
import statistics
import sys
import time

from . import layouts as _lay
from . import opgraph as _og


# --------------------------------------------------------------------------- #
# measuring one configuration
# --------------------------------------------------------------------------- #

class LayerTimer:
    """Runs the layer under a layouts dict on fixed device buffers.

    A layout changes strides, not element counts, so every tensor is allocated
    once; inputs hold i.i.d. values, whose statistics do not depend on the
    order they are read in."""

    def __init__(self, batch_size, max_seq_len, num_heads, embedding_size, intermediate_size=None,
                 activation='relu', p=0.1, iters=5, warmup=2, device='cuda', seed=0x5EED):
        import torch
        from . import _lib
        self.torch, self._lib = torch, _lib
        self.dims = (batch_size, max_seq_len, num_heads, embedding_size)
        self.intermediate_size = intermediate_size or 4 * embedding_size
        self.activation, self.p, self.iters, self.warmup, self.seed = activation, p, iters, warmup, seed
        sizes = _lay.sizes_map(batch_size, max_seq_len, num_heads, embedding_size, self.intermediate_size)
        g = torch.Generator().manual_seed(1234)

        def numel(name):
            n = 1
            for d in _lay.CANONICAL[name]:
                n *= sizes[d]
            return n

        def rand(name, std):
            return (std * torch.randn(numel(name), generator=g)).half().to(device)

        def empty(name):
            return torch.empty(numel(name), dtype=torch.float16, device=device)

        self.buf = {'X': rand('X', 1.0), 'DY': rand('SB2', 1.0), 'Y': empty('SB2'), 'DX': empty('X')}
        for name in _lay.PARAM_NAMES:
            if name in ('S1', 'S2'):
                t = torch.ones(numel(name), dtype=torch.float16, device=device)
            elif name in ('B1', 'B2'):
                t = torch.zeros(numel(name), dtype=torch.float16, device=device)
            else:
                t = rand(name, 0.02)
            self.buf[name] = t
            self.buf['D' + name] = empty(name)
        for name in _lay.FWD_NAMES + _lay.BWD_NAMES:
            self.buf[name] = empty(name)
        self.measurements = 0

    def _handle(self, layouts, profiling):
        b, l, h, e = self.dims
        cfg = self._lib.make_config(b, l, h, e, layouts, self.p, self.p, self.p, self.p,
                                    activation=self.activation, seed=self.seed,
                                    intermediate_size=self.intermediate_size)
        handle = self._lib.Handle(cfg)
        # every tensor in the order under test (by default the library would run a configuration with
        # feature-major activations in its own orders and copy at the boundary)
        handle.set_option(self._lib.OPT_PRIVATE_LAYOUTS, 0)
        handle.set_stream(self.torch.cuda.current_stream().cuda_stream)
        if profiling:
            handle.profile_enable(True)
        return handle

    def _pointers(self, layouts):
        ptr = {k: v.data_ptr() for k, v in self.buf.items()}
        params = [n for n, _ in layouts['params']]
        fwd = [n for n, _ in layouts['forward_interm']]
        bwd = [n for n, _ in layouts['backward_interm']]
        f = [ptr['X']] + [ptr[n] for n in params] + [ptr[n] for n in fwd] + [ptr['Y']]
        b = ([ptr['DY']] + [ptr['D' + n] for n in params] + [ptr[n] for n in bwd]
             + [ptr[n] for n in params] + [ptr[n] for n in fwd] + [ptr['X'], ptr['DX']])
        return (ctypes.c_void_p * len(f))(*f), len(f), (ctypes.c_void_p * len(b))(*b), len(b)

    def usable(self, layouts):
        """False when a contraction cannot be expressed as a GEMM under these layouts
        (einsumparser.h:9-55 has the same limits) or would run on the scalar
        fallback kernel."""
        try:
            handle = self._handle(layouts, False)
        except self._lib.SubstationError:
            return False
        try:
            t = _og.operand_layouts(layouts)
            return all(handle.classify(t[a], t[b], t[c])['kernel'] == 1
                       for a, b, c in _og.EINSUMS.values())
        finally:
            handle.close()

    def measure(self, layouts):
        """operator -> seconds (median over the timed iterations)."""
        lib = self._lib.load()
        handle = self._handle(layouts, True)
        fp, nf, bp, nb = self._pointers(layouts)
        times = {}
        try:
            for it in range(self.warmup + self.iters):
                self._lib.check(lib.sub_encoder_forward(handle.ptr, fp, nf), 'encoder_forward')
                self._lib.check(lib.sub_encoder_backward(handle.ptr, bp, nb), 'encoder_backward')
                prof = handle.profile_read()      # both passes; no host wait between them
                if it >= self.warmup:
                    for name, ms in prof:
                        times.setdefault(name, []).append(ms * 1e-3)
        finally:
            handle.close()
        self.measurements += 1
        return {k: statistics.median(v) for k, v in times.items()}

    def wall(self, layouts, steps=50, warmup=5):
        """Seconds per forward+backward without per-operator timing."""
        torch = self.torch
        lib = self._lib.load()
        handle = self._handle(layouts, False)
        fp, nf, bp, nb = self._pointers(layouts)
        try:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            for it in range(warmup + steps):
                if it == warmup:
                    e0.record()
                self._lib.check(lib.sub_encoder_forward(handle.ptr, fp, nf), 'encoder_forward')
                self._lib.check(lib.sub_encoder_backward(handle.ptr, bp, nb), 'encoder_backward')
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e-3 / steps
        finally:
            handle.close()


# --------------------------------------------------------------------------- #
# the table and the descent
# --------------------------------------------------------------------------- #

class LayoutSearch:
    """Coordinate descent on the measured operator-time table (the place of the shortest-path
    search of config_selection/optimize.py:13-493).

    ``timer`` needs ``measure(layouts) -> {operator: seconds}`` and
    ``usable(layouts) -> bool``."""

    def __init__(self, timer, start, tie_io=True, fixed=(), min_gain=0.002, log=None, out=sys.stdout,
                 budget_s=None, max_compound=4096):
        self.timer, self.tie_io, self.min_gain = timer, tie_io, min_gain
        self.max_compound = max_compound     # largest number of settings one compound coordinate may have
        self.fixed = set(fixed)
        self.current = _lay.validate(_og.with_layouts(start, {}))
        self.table = {}          # (operator, layouts of its tensors) -> seconds, min over measurements
        self.log, self.out = log, out
        self.deadline = None if budget_s is None else time.monotonic() + budget_s
        self.evaluations = 0
        self._last_say = time.monotonic()

    # -- table ------------------------------------------------------------- #
    @staticmethod
    def key_tensors(op):
        """Tensors whose layouts decide an operator's time: its own, and for
        launches that can stand in for one another those of the whole group
        (which of them run depends on all of them; the ones that do not run
        enter 0 s)."""
        for group in _og.ALTERNATIVES:
            if op in group:
                seen = []
                for member in group:
                    seen += [n for n in _og.OP_TENSORS[member] if n not in seen]
                    seen += [n for n in _og.GROUP_ALSO_DEPENDS.get(member, ()) if n not in seen]
                return tuple(seen)
        return _og.OP_TENSORS[op]

    @classmethod
    def _keys(cls, layouts):
        t = _og.tensor_layouts(layouts)
        return {op: (op, tuple(t[n] for n in cls.key_tensors(op))) for op in _og.OP_TENSORS}

    def _enter(self, layouts, times):
        unknown = set(times) - set(_og.OP_TENSORS)
        if unknown:
            raise KeyError(f'timed operators missing from the operator graph: {sorted(unknown)}')
        t = _og.tensor_layouts(layouts)
        for op, k in self._keys(layouts).items():
            if op not in times and not any(op in g for g in _og.ALTERNATIVES):
                raise KeyError(f'operator {op} was not timed')
            sec = times.get(op, 0.0)
            new = k not in self.table
            if new or sec < self.table[k]:
                self.table[k] = sec
            if new and self.log is not None:
                fields = ' '.join(f'{n} = {t[n]}' for n in self.key_tensors(op))
                self.log.write(f'op = {op} {fields} time = {sec:g} s\n')

    def cost(self, layouts, force=False):
        """Summed operator time of a configuration; measured when the table lacks
        one of its entries (or when ``force`` asks for a fresh measurement)."""
        keys = self._keys(layouts)
        if not force and all(k in self.table for k in keys.values()):
            return sum(self.table[k] for k in keys.values())
        if not self.timer.usable(layouts):
            return float('inf')
        times = self.timer.measure(layouts)
        self._timed = set(times)
        self._enter(layouts, times)
        self.evaluations += 1
        if time.monotonic() - self._last_say > 20:
            self._say(f'  ... {self.evaluations} runs, {len(self.table)} table entries')
        return sum(self.table[k] for k in keys.values())

    # -- moves ------------------------------------------------------------- #
    def _expand(self, changes):
        """Applies the input/output tie and drops fixed tensors."""
        ch = dict(changes)
        if self.tie_io:
            if 'X' in ch:
                ch['SB2'] = ch['X']
            elif 'SB2' in ch:
                ch['X'] = ch['SB2']
        if any(n in self.fixed for n in ch):
            return None
        return ch

    def moves(self):
        """Yields (label, [changes, ...]): each entry is one coordinate with its
        alternative settings."""
        names = [n for n in _og.searchable_tensors() if n not in self.fixed]
        if self.tie_io:
            names = [n for n in names if n != 'SB2']
        seen = set()

        def group_moves(label, members):
            members = [m for m in members if len(_og.candidate_layouts(m)) > 1]
            if len(members) < 2:
                return None
            key = tuple(sorted(members))
            if key in seen:
                return None
            seen.add(key)
            alts = []
            # members share one dim set, except that stacked tensors lead with Q
            base = _lay.CANONICAL[members[0]].replace('Q', '')
            for p in itertools.permutations(base):
                p = ''.join(p)
                alts.append({m: ('Q' + p if 'Q' in _lay.CANONICAL[m] else p) for m in members})
            return label, alts

        def dimset(n):
            return ''.join(sorted(_lay.CANONICAL[n].replace('Q', '')))

        # 1. whole classes of same-shaped tensors
        classes = {}
        for n in names + (['SB2'] if self.tie_io else []):
            classes.setdefault(dimset(n), []).append(n)
        for ds, members in classes.items():
            gm = group_moves(f'class {ds}', members)
            if gm:
                yield gm
        # 1b. a class together with the weights of the operators that touch it, every combination of
        # their layouts as one coordinate.  What switches a fused path on or off is a property of such
        # a group -- the attention kernels with the scores in registers need the projections, their
        # gradients, WKQV, BKQV and WO to agree on where heads and head size lie; the activation
        # epilogues need the [B,J,U] tensors and LINW1 / LINW2 to agree -- and no path of single-coordinate
        # improvements leads from one such family of layouts to another: half-way configurations cannot be
        # expressed as GEMMs at all or fall to strided kernels.
        for ds, members in classes.items():
            members = [m for m in members if len(_og.candidate_layouts(m)) > 1]
            params = []
            for _, _, tensors in _og.OPERATORS:
                if any(m in tensors for m in members):
                    params += [n for n in tensors if n in _lay.PARAM_NAMES and n not in params
                               and n not in self.fixed and len(_og.candidate_layouts(n)) > 1]
            if not members or not params:
                continue
            count = len(list(itertools.permutations(_lay.CANONICAL[members[0]].replace('Q', ''))))
            for n in params:
                count *= len(_og.candidate_layouts(n))
            if count > self.max_compound:
                continue
            base = _lay.CANONICAL[members[0]].replace('Q', '')
            alts = []
            for p in itertools.permutations(base):
                p = ''.join(p)
                act = {m: ('Q' + p if 'Q' in _lay.CANONICAL[m] else p) for m in members}
                for combo in itertools.product(*[_og.candidate_layouts(n) for n in params]):
                    alts.append({**act, **dict(zip(params, combo))})
            yield f'class {ds} with ' + ' '.join(params), alts
        # 2. same-shaped tensors of one operator
        for op, _, tensors in _og.OPERATORS:
            per = {}
            for n in tensors:
                if n in self.fixed:
                    continue
                per.setdefault(dimset(n), []).append(n)
            for ds, members in per.items():
                gm = group_moves(f'{op} {ds}', members)
                if gm:
                    yield gm
        # 3. single tensors
        for n in names:
            yield n, [{n: l} for l in _og.candidate_layouts(n)]

    # -- descent ----------------------------------------------------------- #
    def _say(self, msg):
        self._last_say = time.monotonic()
        print(msg, file=self.out, flush=True)

    def out_of_time(self):
        return self.deadline is not None and time.monotonic() > self.deadline

    def run(self, sweeps=3):
        cur_cost = self.cost(self.current, force=True)
        if cur_cost == float('inf'):
            raise ValueError('the starting configuration is not usable')
        self._say(f'start: {cur_cost * 1e6:.1f} us summed operator time')
        for sweep in range(sweeps):
            improved = False
            for label, alts in self.moves():
                if self.out_of_time():
                    self._say('time budget used up')
                    return self.current
                best, best_cost = None, cur_cost
                for raw in alts:
                    if self.out_of_time():
                        break
                    ch = self._expand(raw)
                    if ch is None:
                        continue
                    cand = _og.with_layouts(self.current, ch)
                    if _og.tensor_layouts(cand) == _og.tensor_layouts(self.current):
                        continue
                    c = self.cost(cand)
                    if c < best_cost:
                        best, best_cost = cand, c
                if best is None or best_cost > cur_cost * (1 - self.min_gain):
                    continue
                # confirm on fresh measurements of both before moving
                c_new = self.cost(best, force=True)
                c_old = self.cost(self.current, force=True)
                if c_new <= c_old * (1 - self.min_gain):
                    diff = {n: l for n, l in _og.tensor_layouts(best).items()
                            if _og.tensor_layouts(self.current)[n] != l}
                    self._say(f'sweep {sweep} {label}: {c_old * 1e6:.1f} -> {c_new * 1e6:.1f} us  '
                              + ' '.join(f'{n}:{l}' for n, l in diff.items())
                              + f'  [{self.evaluations} runs]')
                    self.current, cur_cost, improved = best, c_new, True
                else:
                    cur_cost = c_old
            self._say(f'sweep {sweep} done: {cur_cost * 1e6:.1f} us, {self.evaluations} runs, '
                      f'{len(self.table)} table entries')
            if not improved:
                break
        return self.current

    def report(self, layouts):
        """Per-operator table of a configuration, like print_configurations of
        config_selection/optimize.py:419-440."""
        t = _og.tensor_layouts(layouts)
        tot = {'fwd': 0.0, 'bwd': 0.0}
        keys = self._keys(layouts)
        for op, which, tensors in _og.OPERATORS:
            sec = self.table.get(keys[op])
            if sec is None or (sec == 0.0 and op not in self._timed):
                continue
            best = min(v for (o, _), v in self.table.items() if o == op)
            tot[which] += sec
            lay = ' '.join(f'{n}={t[n]}' for n in tensors)
            self._say(f'{op}: {lay} | Time: {sec:g} (from best: {sec - best:g})')
        self._say(f"Forward time: {tot['fwd']:g} | Backward time: {tot['bwd']:g} | "
                  f"Total: {tot['fwd'] + tot['bwd']:g}")


# --------------------------------------------------------------------------- #
# one operator under all its layouts
# --------------------------------------------------------------------------- #

class OperatorSweep:
    """One fused operator timed on its own under every layout of its tensors: the
    counterpart of the per-kernel sweep of pytorch_module/benchmark.py:178-302,
    1362-1472, whose results the reference ships as perf_softmax.txt, perf_bsb.txt,
    perf_bdrln.txt, perf_bad.txt.  The reference compiles one kernel per
    combination; strides are run-time data here, so a combination is one call
    through the operator entry points of the C ABI.  Tensors are grouped into
    roles that change layout together (as the reference's files do: softmax
    ``IN -> OUT``); every role runs through all permutations of its dims."""

    #: operator -> (dims, [(role, [tensor arguments])]): arguments named as in substation_amd.ops.Ops
    OPERATORS = {
        'softmax': ('HBJK', [('IN', ['beta', 'drop']), ('OUT', ['alpha', 'mask'])]),
        'bs': ('HBJK', [('IN', ['alpha', 'mask', 'ddrop']), ('OUT', ['dbeta'])]),
        'bdrln': ('BJI', [('IN', ['inp', 'resid']), ('OUT', ['lin', 'mask', 'diff', 'normed', 'out'])]),
        'blnrd': ('BJI', [('IN', ['dout', 'diff', 'mask']), ('OUT', ['d_ln_in', 'd_drop_in'])]),
        'bad': ('BJU', [('IN', ['inp']), ('OUT', ['lin', 'mask', 'out'])]),
        'bdrlb': ('BJU', [('IN', ['ddrop', 'mask', 'lin']), ('OUT', ['dlinear'])]),
        'bsb': ('BJI', [('IN', ['inp', 'dout']), ('DIN', ['din'])]),
        'ebsb': ('BJI', [('IN', ['inp', 'dout1', 'dout2', 'dlinear']), ('DIN', ['din'])]),
        'baob': ('BJI', [('IN', ['datt'])]),
        'bei': ('BJI', [('IN', ['dxatt', 'dresid1']), ('OUT', ['dx'])]),
    }

    def __init__(self, batch, seq, heads, embed, intermediate=None, iters=5, warmup=2, device='cuda'):
        import torch
        from . import ops as _ops
        self.torch = torch
        self.o = _ops.Ops(batch, seq, heads, embed, intermediate_size=intermediate, seed=0x5EED)
        self.iters, self.warmup, self.device = iters, warmup, device
        self.g = torch.Generator(device=device).manual_seed(7)

    def _tensor(self, layout, kind='normal'):
        t = self.o.empty(layout, self.device)
        if kind == 'mask':
            t.copy_((self.torch.rand(t.shape, device=self.device, generator=self.g) >= 0.1).half())
        elif kind == 'positive':
            t.normal_(0.0, 1.0, generator=self.g).abs_().add_(0.5)
        else:
            t.normal_(0.0, 1.0, generator=self.g)
        return t

    def _vector(self, dim):
        n = self.o.sizes[dim]
        return self.torch.empty(n, dtype=self.torch.float16, device=self.device).normal_(0.0, 0.1, generator=self.g)

    def _call(self, op, lay):
        """Allocates the operator's tensors under ``lay`` (argument -> layout) and returns a
        function that launches it once."""
        o, T = self.o, self._tensor
        if op == 'softmax':
            a = dict(beta=T(lay['beta']), alpha=T(lay['alpha']), mask=T(lay['mask']), drop=T(lay['drop']))
            return lambda: o.softmax(a['beta'], lay['beta'], a['alpha'], lay['alpha'], a['mask'], lay['mask'],
                                     a['drop'], lay['drop'], scale=0.125, p=0.1)
        if op == 'bs':
            a = dict(alpha=T(lay['alpha']), mask=T(lay['mask'], 'mask'), ddrop=T(lay['ddrop']), dbeta=T(lay['dbeta']))
            return lambda: o.bs(a['alpha'], lay['alpha'], a['mask'], lay['mask'], a['ddrop'], lay['ddrop'],
                                a['dbeta'], lay['dbeta'], scale=0.125)
        if op == 'bdrln':
            a = {k: T(lay[k]) for k in ('inp', 'resid', 'lin', 'mask', 'diff', 'normed', 'out')}
            istd, v = T('BJ'), [self._vector('I') for _ in range(3)]
            return lambda: o.bdrln(a['inp'], lay['inp'], a['resid'], lay['resid'], v[0], v[1], v[2], a['lin'], lay['lin'],
                                   a['mask'], lay['mask'], a['diff'], lay['diff'], a['normed'], lay['normed'],
                                   a['out'], lay['out'], istd, 'BJ', p=0.1, site=1)
        if op == 'blnrd':
            a = dict(dout=T(lay['dout']), diff=T(lay['diff']), mask=T(lay['mask'], 'mask'), d_ln_in=T(lay['d_ln_in']),
                     d_drop_in=T(lay['d_drop_in']))
            istd = T('BJ', 'positive')
            return lambda: o.blnrd(a['dout'], lay['dout'], istd, 'BJ', a['diff'], lay['diff'], a['mask'], lay['mask'],
                                   a['d_ln_in'], lay['d_ln_in'], a['d_drop_in'], lay['d_drop_in'])
        if op == 'bad':
            a = {k: T(lay[k]) for k in ('inp', 'lin', 'mask', 'out')}
            b = self._vector('U')
            return lambda: o.bad(a['inp'], lay['inp'], b, a['lin'], lay['lin'], a['mask'], lay['mask'], a['out'],
                                 lay['out'], p=0.1, site=2)
        if op == 'bdrlb':
            a = dict(ddrop=T(lay['ddrop']), mask=T(lay['mask'], 'mask'), lin=T(lay['lin']), dlinear=T(lay['dlinear']))
            db = self._vector('U')
            return lambda: o.bdrlb(a['ddrop'], lay['ddrop'], a['mask'], lay['mask'], a['lin'], lay['lin'],
                                   a['dlinear'], lay['dlinear'], db)
        if op == 'bsb':
            a = {k: T(lay[k]) for k in ('inp', 'dout', 'din')}
            v = [self._vector('I') for _ in range(3)]
            return lambda: o.bsb(a['inp'], lay['inp'], v[0], a['dout'], lay['dout'], a['din'], lay['din'], v[1], v[2])
        if op == 'ebsb':
            a = {k: T(lay[k]) for k in ('inp', 'dout1', 'dout2', 'dlinear', 'din')}
            v = [self._vector('I') for _ in range(4)]
            return lambda: o.ebsb(a['inp'], lay['inp'], v[0], a['dout1'], lay['dout1'], a['dout2'], lay['dout2'],
                                  a['dlinear'], lay['dlinear'], a['din'], lay['din'], v[1], v[2], v[3])
        if op == 'baob':
            a, v = T(lay['datt']), self._vector('I')
            return lambda: o.baob(a, lay['datt'], v)
        if op == 'bei':
            a = {k: T(lay[k]) for k in ('dxatt', 'dresid1', 'dx')}
            return lambda: o.bei(a['dxatt'], lay['dxatt'], a['dresid1'], lay['dresid1'], a['dx'], lay['dx'])
        raise KeyError(op)

    def time(self, op, role_layouts):
        """Seconds per launch with every tensor of a role in that role's layout."""
        torch = self.torch
        _, roles = self.OPERATORS[op]
        lay = {arg: role_layouts[role] for role, args in roles for arg in args}
        run = self._call(op, lay)
        for _ in range(self.warmup):
            run()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(self.iters):
            run()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / self.iters

    def sweep(self, op, out=sys.stdout, budget_s=None):
        """Every combination of role layouts; one line per combination, `op ROLE layout ... time = X s`
        (the key = value ... time = X s lines of pytorch_module/benchmark.py:1437-1447).  Returns the
        list of (role_layouts, seconds), fastest first."""
        dims, roles = self.OPERATORS[op]
        perms = [''.join(p) for p in itertools.permutations(dims)]
        results = []
        t0 = time.monotonic()
        for combo in itertools.product(perms, repeat=len(roles)):
            if budget_s is not None and time.monotonic() - t0 > budget_s:
                print(f'# time budget used up after {len(results)} combinations', file=out, flush=True)
                break
            rl = {role: l for (role, _), l in zip(roles, combo)}
            sec = self.time(op, rl)
            results.append((rl, sec))
            print(f'op = {op} ' + ' '.join(f'{r} = {l}' for r, l in rl.items()) + f' time = {sec:g} s', file=out,
                  flush=True)
        results.sort(key=lambda x: x[1])
        return results


def _start_layouts(name):
    if name == 'mi355x':
        return _lay.mi355x_layouts()
    if name in ('bert-b8-l512-h16-e1024', 'bert-b96-l128-h16-e1024'):
        return _lay.reference_layouts(name)
    return _lay.load_layouts(name)


def main(argv=None):
    ap = argparse.ArgumentParser(description='Find layouts for the encoder layer from MI355X timings.')
    ap.add_argument('--batch', type=int, default=8)
    ap.add_argument('--seq', type=int, default=512)
    ap.add_argument('--heads', type=int, default=16)
    ap.add_argument('--embed', type=int, default=1024)
    ap.add_argument('--intermediate', type=int, default=None)
    ap.add_argument('--activation', default='relu', choices=['relu', 'gelu'])
    ap.add_argument('--start', default='mi355x',
                    help="'mi355x', a shipped reference configuration name, or a layouts pickle")
    ap.add_argument('--sweeps', type=int, default=3)
    ap.add_argument('--iters', type=int, default=5)
    ap.add_argument('--budget-s', type=float, default=None, help='stop moving after this many seconds')
    ap.add_argument('--fix', nargs='*', default=[], help='tensors whose layout must not change')
    ap.add_argument('--free-io', action='store_true',
                    help='let input and output layouts differ (layers then no longer stack)')
    ap.add_argument('--min-gain', type=float, default=0.002)
    ap.add_argument('--out', default=None, help='layouts pickle to write')
    ap.add_argument('--log', default=None, help="table entries as 'k = v ... time = X s' lines")
    ap.add_argument('--sweep-op', default=None, choices=sorted(OperatorSweep.OPERATORS),
                    help='time this one operator on its own under every layout of its tensors instead of '
                         'searching (lines go to --log or stdout)')
    args = ap.parse_args(argv)

    if args.sweep_op:
        sweep = OperatorSweep(args.batch, args.seq, args.heads, args.embed, args.intermediate, iters=args.iters)
        log = open(args.log, 'w') if args.log else sys.stdout
        try:
            res = sweep.sweep(args.sweep_op, out=log, budget_s=args.budget_s)
        finally:
            if args.log:
                log.close()
        show = lambda r: ' '.join(f'{k} {v}' for k, v in r[0].items()) + f' {r[1] * 1e6:.2f} us'
        print(f'{args.sweep_op}: {len(res)} combinations; best {show(res[0])}; worst {show(res[-1])}', flush=True)
        return res

    start = _start_layouts(args.start)
    timer = LayerTimer(args.batch, args.seq, args.heads, args.embed, args.intermediate,
                       activation=args.activation, iters=args.iters)
    log = open(args.log, 'w') if args.log else None
    try:
        search = LayoutSearch(timer, start, tie_io=not args.free_io, fixed=args.fix,
                              min_gain=args.min_gain, log=log, budget_s=args.budget_s)
        best = search.run(args.sweeps)
        search.report(best)
    finally:
        if log:
            log.close()
    w0, w1 = timer.wall(start), timer.wall(best)
    print(f'forward+backward, no per-operator timing: start {w0 * 1e3:.4f} ms, found {w1 * 1e3:.4f} ms',
          flush=True)
    if w1 > w0:
        print('the found configuration is not faster end to end; keeping the start', flush=True)
        best = start
    if args.out:
        _lay.save_layouts(best, args.out)
        print('wrote', args.out, flush=True)
    for key in ('input', 'output'):
        print(key, best[key])
    for key in ('params', 'forward_interm', 'backward_interm'):
        print(key, ' '.join(f'{n}:{l}' for n, l in best[key]))
    return best


if __name__ == '__main__':
    main()
