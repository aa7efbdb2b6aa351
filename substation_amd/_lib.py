"""ctypes binding of libsubstation_amd.so (declared in include/substation_amd.h).

Takes the place of the ``ctypes.CDLL`` block at pytorch_module/encoder.py:395-403.
There is no CPU fallback: if the library is missing, loading raises."""
import ctypes
import os

from . import layouts as _lay

HERE = os.path.dirname(os.path.abspath(__file__))
#: the in-tree build; SUBSTATION_AMD_LIB names another build of the same sources
LIB_PATH = os.environ.get('SUBSTATION_AMD_LIB') or os.path.join(HERE, 'lib', 'libsubstation_amd.so')

N_PARAMS, N_FWD, N_BWD = 12, 23, 14
ABI_VERSION = 1
ACTIVATIONS = {'relu': 0, 'gelu': 1}
OPT_FUSE_EPILOGUES = 1
OPT_FUSE_LN_BACKWARD = 2
OPT_FUSE_SCORES = 3
OPT_FUSE_ATTENTION = 4
OPT_PAIR_PRODUCTS = 5
OPT_RELU_FROM_OUTPUT = 6
OPT_FINISH_IN_PAIR = 7
OPT_SIDE_JOBS = 8
OPT_PACKED_MASKS = 9
OPT_SKIP_UNREAD = 10
OPT_PRIVATE_LAYOUTS = 11
FUSE_REQUIRED = 2


class SubConfig(ctypes.Structure):
    _fields_ = [
        ('abi_version', ctypes.c_int32),
        ('batch', ctypes.c_int32), ('seq', ctypes.c_int32), ('heads', ctypes.c_int32),
        ('embed', ctypes.c_int32), ('intermediate', ctypes.c_int32),
        ('dtype', ctypes.c_int32), ('activation', ctypes.c_int32),
        ('p_softmax', ctypes.c_float), ('p_resid1', ctypes.c_float),
        ('p_act', ctypes.c_float), ('p_resid2', ctypes.c_float),
        ('ln_eps', ctypes.c_float),
        ('seed', ctypes.c_uint64),
        ('input_layout', ctypes.c_char_p), ('output_layout', ctypes.c_char_p),
        ('param_names', ctypes.c_char_p * N_PARAMS), ('param_layouts', ctypes.c_char_p * N_PARAMS),
        ('fwd_names', ctypes.c_char_p * N_FWD), ('fwd_layouts', ctypes.c_char_p * N_FWD),
        ('bwd_names', ctypes.c_char_p * N_BWD), ('bwd_layouts', ctypes.c_char_p * N_BWD),
    ]


_lib = None

_VP, _CP, _F, _U32, _U64, _I = (ctypes.c_void_p, ctypes.c_char_p, ctypes.c_float, ctypes.c_uint32,
                                ctypes.c_uint64, ctypes.c_int)

#: every symbol include/substation_amd.h declares: name -> (restype, argtypes)
SIGNATURES = {
    'init': (_VP, []),
    'destroy': (None, [_VP]),
    'encoder_forward': (_I, [_VP] * (1 + 1 + N_PARAMS + N_FWD + 1)),
    'encoder_backward': (_I, [_VP] * (1 + 1 + N_PARAMS + N_BWD + N_PARAMS + N_FWD + 1 + 1)),
    'init_cfg': (_VP, [ctypes.POINTER(SubConfig)]),
    'sub_configure': (_I, [_VP, ctypes.POINTER(SubConfig)]),
    'sub_set_stream': (_I, [_VP, _VP]),
    'sub_set_rng': (_I, [_VP, _U64, _U32]),
    'sub_set_rng_counter': (_I, [_VP, _VP]),
    'sub_last_error': (_CP, []),
    'sub_set_option': (_I, [_VP, _I, _I]),
    'sub_ops_defer': (_I, [_VP, _I]),
    'sub_get_option': (_I, [_VP, ctypes.c_int, ctypes.POINTER(ctypes.c_int)]),
    'sub_tensor_layout': (_I, [_VP, ctypes.c_char_p, ctypes.c_char_p]),
    'sub_attention_in_registers': (_I, [_VP, ctypes.POINTER(_I)]),
    'sub_encoder_forward': (_I, [_VP, ctypes.POINTER(_VP), _I]),
    'sub_encoder_backward': (_I, [_VP, ctypes.POINTER(_VP), _I]),
    'sub_profile_enable': (_I, [_VP, _I]),
    'sub_profile_read': (_I, [_VP, _I, ctypes.POINTER(_CP), ctypes.POINTER(_F)]),
    'sub_profile_read_clocks': (_I, [_VP, _I, ctypes.POINTER(_CP), ctypes.POINTER(_F)]),
    'sub_op_softmax': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _F, _F, _U32]),
    'sub_op_softmax_masked': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _F, _F, _F, _U32]),
    'sub_set_attention_mask': (_I, [_VP, _VP, _CP]),
    'sub_op_attention_forward': (_I, [_VP, _I, _I, _VP, _CP, _VP, _VP, _CP, _VP, _CP, _VP, _VP, _VP, _CP,
                                      _F, _F, _U32]),
    'sub_op_attention_backward': (_I, [_VP, _I, _I, _VP, _CP, _VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _VP,
                                       _VP, _CP, _VP, _VP, _CP, _VP, _CP, _F]),
    'sub_op_attention_backward_biases': (_I, [_VP, _I, _I, _VP, _CP, _VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _VP,
                                              _VP, _CP, _VP, _VP, _CP, _VP, _CP, _F, _VP, _VP, _VP]),
    'sub_op_bs': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _F]),
    'sub_op_bdrln': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _VP, _VP, _VP, _CP, _VP, _CP, _VP, _CP,
                          _VP, _CP, _VP, _CP, _VP, _CP, _F, _U32]),
    'sub_op_blnrd': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP]),
    'sub_op_bad': (_I, [_VP, _VP, _CP, _VP, _VP, _CP, _VP, _CP, _VP, _CP, _F, _U32]),
    'sub_op_bsb': (_I, [_VP, _VP, _CP, _VP, _VP, _CP, _VP, _CP, _VP, _VP]),
    'sub_op_ebsb': (_I, [_VP, _VP, _CP, _VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _VP, _VP]),
    'sub_op_bdrlb': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _VP]),
    'sub_op_baob': (_I, [_VP, _VP, _CP, _VP]),
    'sub_op_aib': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP]),
    'sub_op_baib': (_I, [_VP, _VP, _CP, _VP, _CP]),
    'sub_op_bei': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP]),
    'sub_op_relayout': (_I, [_VP, _VP, _CP, _VP, _CP]),
    'sub_probe_fetch': (_I, [_VP, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, _VP, ctypes.POINTER(ctypes.c_float),
                        ctypes.POINTER(ctypes.c_float)]),
    'sub_op_ln_backward': (_I, [_VP, ctypes.c_int, _VP, _CP, _VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP,
                                _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _VP, _VP, _VP]),
    'sub_op_ln_backward_static': (_I, [_VP, ctypes.c_int, _VP, _CP, _VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _VP,
                                       _CP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _VP, _VP, _VP]),
    'sub_op_einsum': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP, _F]),
    'sub_op_einsum_add': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _F]),
    'sub_op_einsum_bad': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _VP, _CP, _VP, _F, _U32,
                               ctypes.POINTER(ctypes.c_int)]),
    'sub_op_einsum_bdrlb': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _VP, _CP, _VP,
                                 ctypes.POINTER(ctypes.c_int)]),
    'sub_op_einsum_pair': (_I, [_VP, _VP, _CP, _VP, _CP, _VP, _CP, _VP, _CP, _F,
                                _VP, _CP, _VP, _CP, _VP, _CP, _F, ctypes.POINTER(ctypes.c_int)]),
    'sub_layout_strides': (_I, [_VP, _CP, ctypes.POINTER(ctypes.c_int64)]),
    'sub_einsum_classify': (_I, [_VP, _CP, _CP, _CP, ctypes.POINTER(ctypes.c_int64)]),
    'sub_philox_fields_host': (_I, [_U64, _U32, _U32, _U64, _U64, ctypes.POINTER(ctypes.c_uint16)]),
    'sub_dropout_threshold': (_U32, [_F]),
}


def load():
    """Loads the prebuilt library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f'{LIB_PATH} is missing: build it with `python -m substation_amd.build` '
            '(there is no fallback implementation)')
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class SubstationError(RuntimeError):
    pass


def check(rc, what=''):
    if rc is not None and rc < 0:
        msg = load().sub_last_error()
        raise SubstationError((what + ': ' if what else '') + (msg.decode() if msg else 'unknown error'))
    return rc


def make_config(batch_size, max_seq_len, num_heads, embedding_size, layouts, p_softmax=0.0,
                p_resid1=0.0, p_act=0.0, p_resid2=0.0, activation='relu', seed=0,
                intermediate_size=0, ln_eps=0.0):
    """Builds a sub_config from a layouts dict (names/layouts in the dict's own
    order, which is also the order the pointers are passed in)."""
    _lay.validate(layouts)
    if activation not in ACTIVATIONS:
        raise ValueError('Unknown activation ' + str(activation))
    c = SubConfig()
    c.abi_version = ABI_VERSION
    c.batch, c.seq, c.heads, c.embed = batch_size, max_seq_len, num_heads, embedding_size
    c.intermediate = intermediate_size or 0
    c.dtype = 0
    c.activation = ACTIVATIONS[activation]
    c.p_softmax, c.p_resid1, c.p_act, c.p_resid2 = p_softmax, p_resid1, p_act, p_resid2
    c.ln_eps = ln_eps
    c.seed = seed
    c.input_layout = layouts['input'][1].encode()
    c.output_layout = layouts['output'][1].encode()
    for key, names, lays in (('params', c.param_names, c.param_layouts),
                             ('forward_interm', c.fwd_names, c.fwd_layouts),
                             ('backward_interm', c.bwd_names, c.bwd_layouts)):
        for i, (n, l) in enumerate(layouts[key]):
            names[i] = n.encode()
            lays[i] = l.encode()
    return c


class Handle:
    """Owns one native encoder handle."""

    def __init__(self, config):
        self.lib = load()
        self._config = config       # keeps the char buffers alive
        self.ptr = self.lib.init_cfg(ctypes.byref(config))
        if not self.ptr:
            msg = self.lib.sub_last_error()
            raise SubstationError('init_cfg: ' + (msg.decode() if msg else 'failed'))

    def close(self):
        if getattr(self, 'ptr', None):
            self.lib.destroy(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_stream(self, stream):
        check(self.lib.sub_set_stream(self.ptr, ctypes.c_void_p(stream)), 'sub_set_stream')

    def set_rng(self, seed, step=0):
        check(self.lib.sub_set_rng(self.ptr, seed, step), 'sub_set_rng')

    def set_rng_counter(self, device_ptr):
        check(self.lib.sub_set_rng_counter(self.ptr, ctypes.c_void_p(device_ptr or 0)), 'sub_set_rng_counter')

    def set_attention_mask(self, device_ptr, layout='JK'):
        check(self.lib.sub_set_attention_mask(self.ptr, ctypes.c_void_p(device_ptr or 0), layout.encode()),
              'sub_set_attention_mask')

    def defer_column_sums(self, on):
        """sub_ops_defer: between on=True and on=False the operators' column sums are finished by one launch."""
        check(self.lib.sub_ops_defer(self.ptr, 1 if on else 0), 'sub_ops_defer')

    def set_option(self, option, value):
        check(self.lib.sub_set_option(self.ptr, option, value), 'sub_set_option')

    def get_option(self, option):
        v = ctypes.c_int(0)
        check(self.lib.sub_get_option(self.ptr, option, ctypes.byref(v)), 'sub_get_option')
        return v.value

    def attention_in_registers(self):
        """True when self-attention will run with the scores kept in registers."""
        out = _I(0)
        check(self.lib.sub_attention_in_registers(self.ptr, ctypes.byref(out)), 'sub_attention_in_registers')
        return bool(out.value)

    def tensor_layout(self, name):
        """The dimension order in which the layer calls hold tensor ``name`` inside its buffer: the
        configured one, or the library's own under OPT_PRIVATE_LAYOUTS."""
        out = ctypes.create_string_buffer(16)
        check(self.lib.sub_tensor_layout(self.ptr, name.encode(), out), 'sub_tensor_layout')
        return out.value.decode()

    def profile_enable(self, on=True):
        """on: False / True, or 2 for per-launch timing plus clock samples (profile_read_clocks)."""
        check(self.lib.sub_profile_enable(self.ptr, int(on)), 'sub_profile_enable')

    def profile_read_clocks(self, cap=64):
        """(launch name, shader clock in MHz during it) for the launches profile_read lists."""
        names = (ctypes.c_char_p * cap)()
        mhz = (ctypes.c_float * cap)()
        n = check(self.lib.sub_profile_read_clocks(self.ptr, cap, names, mhz), 'sub_profile_read_clocks')
        return [(names[i].decode(), float(mhz[i])) for i in range(min(n, cap))]

    def profile_read(self, cap=64):
        names = (ctypes.c_char_p * cap)()
        ms = (ctypes.c_float * cap)()
        n = check(self.lib.sub_profile_read(self.ptr, cap, names, ms), 'sub_profile_read')
        return [(names[i].decode(), float(ms[i])) for i in range(min(n, cap))]

    def strides(self, layout):
        out = (ctypes.c_int64 * 8)()
        check(self.lib.sub_layout_strides(self.ptr, layout.encode(), out), 'sub_layout_strides')
        return dict(zip('BJKHPIUQ', out))

    def classify(self, la, lb, lc):
        out = (ctypes.c_int64 * 32)()
        check(self.lib.sub_einsum_classify(self.ptr, la.encode(), lb.encode(), lc.encode(), out),
              'sub_einsum_classify')
        keys = ('batch', 'M', 'N', 'K', 'sAM', 'sAK', 'sAB', 'sBN', 'sBK', 'sBB', 'sCM', 'sCN', 'sCB',
                'nbatch', 'K0', 'sAK0', 'sBK0', 'kernel')
        d = dict(zip(keys, out))
        d['nb'] = list(out[18:21]); d['sAb'] = list(out[21:24]); d['sBb'] = list(out[24:27])
        d['sCb'] = list(out[27:30]); d['K1'] = out[30]
        return d


def philox_fields_host(seed, site, step, start, n):
    import numpy as np
    out = np.empty(n, dtype=np.uint16)
    check(load().sub_philox_fields_host(seed, site, step, start, n,
                                        out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16))))
    return out
