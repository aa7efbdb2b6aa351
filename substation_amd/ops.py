"""Single fused operators and the einsum contraction on torch tensors.

The units pytorch_module/benchmark.py generates, compiles and times one by one
(`Kernel` subclasses at benchmark.py:318-1325); here they are entry points of the
prebuilt library.  Every tensor argument is a contiguous fp16 CUDA tensor whose
dimension order is given by the layout string that follows it.
"""
import contextlib
import ctypes

import torch

from . import _lib
from . import layouts as _lay


def _p(t):
    if t is None:
        return None
    if not (t.is_cuda and t.is_contiguous() and t.dtype == torch.float16):
        raise ValueError('operators take contiguous fp16 CUDA tensors')
    return ctypes.c_void_p(t.data_ptr())


def _s(layout):
    return layout.encode()


class Ops:
    """Operators bound to one problem size (B, L, H, E[, U])."""

    def __init__(self, batch_size, max_seq_len, num_heads, embedding_size, activation='relu',
                 seed=0, intermediate_size=None):
        cfg = _lib.make_config(batch_size, max_seq_len, num_heads, embedding_size,
                               _lay.mi355x_layouts(), activation=activation, seed=seed,
                               intermediate_size=intermediate_size or 0)
        self.handle = _lib.Handle(cfg)
        self.lib = self.handle.lib
        self.sizes = _lay.sizes_map(batch_size, max_seq_len, num_heads, embedding_size,
                                    intermediate_size)

    def _pre(self):
        self.handle.set_stream(torch.cuda.current_stream().cuda_stream)
        return self.handle.ptr

    def empty(self, layout, device='cuda'):
        return torch.empty(_lay.shape_of(layout, self.sizes), dtype=torch.float16, device=device)

    def set_rng(self, seed, step=0):
        self.handle.set_rng(seed, step)

    @contextlib.contextmanager
    def deferred_column_sums(self):
        """Inside the block the operators that reduce over tokens (bsb, ebsb, bdrlb, baob,
        ln_backward) leave the second stage of their column sums to one launch issued
        when the block ends: their bias and scale gradients are complete only then."""
        self._pre()
        self.handle.defer_column_sums(True)
        try:
            yield self
        finally:
            self._pre()
            self.handle.defer_column_sums(False)

    def softmax(self, beta, l_beta, alpha, l_alpha, mask, l_mask, drop, l_drop, scale=1.0, p=0.0,
                site=0, attn_mask=None, l_attn_mask='JK', mask_scale=1.0):
        if attn_mask is not None:
            _lib.check(self.lib.sub_op_softmax_masked(
                self._pre(), _p(beta), _s(l_beta), _p(alpha), _s(l_alpha), _p(mask), _s(l_mask), _p(drop),
                _s(l_drop), _p(attn_mask), _s(l_attn_mask), scale, mask_scale, p, site), 'softmax')
            return
        _lib.check(self.lib.sub_op_softmax(self._pre(), _p(beta), _s(l_beta), _p(alpha), _s(l_alpha),
                                           _p(mask), _s(l_mask), _p(drop), _s(l_drop), scale, p, site),
                   'softmax')

    def attention_workspace(self, n_queries, n_keys, device='cuda'):
        """(stats, keep): what attention_forward hands to attention_backward."""
        rows = self.sizes['H'] * self.sizes['B'] * n_queries
        return (torch.empty(2 * rows, dtype=torch.float32, device=device),
                torch.empty(rows * (n_keys // 32), dtype=torch.int32, device=device))

    def attention_forward(self, q, l_q, k, v, l_kv, out, l_out, stats, keep, scale, p=0.0, site=0,
                          attn_mask=None, l_attn_mask='JK'):
        """out = dropout(softmax(scale * (q.k^T + attn_mask))) . v with the scores in
        registers; the numbers of query and key positions are read off the tensors."""
        nq, nk = q.shape[l_q.index('J')], k.shape[l_kv.index('K')]
        _lib.check(self.lib.sub_op_attention_forward(
            self._pre(), nq, nk, _p(q), _s(l_q), _p(k), _p(v), _s(l_kv), _p(out), _s(l_out),
            ctypes.c_void_p(stats.data_ptr()), ctypes.c_void_p(keep.data_ptr()), _p(attn_mask), _s(l_attn_mask),
            scale, p, site), 'attention_forward')

    def attention_backward(self, q, l_q, k, v, l_kv, out, l_out, d_out, l_dout, stats, keep, dq, l_dq, dk, dv,
                           l_dkv, scale, attn_mask=None, l_attn_mask='JK', dq_bias=None, dk_bias=None, dv_bias=None):
        """``dq_bias``, ``dk_bias``, ``dv_bias``: optional [H, P] outputs, the sums of dq, dk, dv over samples
        and positions (the gradients of the projection biases), formed in the same launches."""
        nq, nk = q.shape[l_q.index('J')], k.shape[l_kv.index('K')]
        _lib.check(self.lib.sub_op_attention_backward_biases(
            self._pre(), nq, nk, _p(q), _s(l_q), _p(k), _p(v), _s(l_kv), _p(out), _s(l_out), _p(d_out),
            _s(l_dout), ctypes.c_void_p(stats.data_ptr()), ctypes.c_void_p(keep.data_ptr()), _p(dq), _s(l_dq),
            _p(dk), _p(dv), _s(l_dkv), _p(attn_mask), _s(l_attn_mask), scale, _p(dq_bias), _p(dk_bias),
            _p(dv_bias)), 'attention_backward')

    def bs(self, alpha, l_alpha, mask, l_mask, ddrop, l_ddrop, dbeta, l_dbeta, scale=1.0):
        _lib.check(self.lib.sub_op_bs(self._pre(), _p(alpha), _s(l_alpha), _p(mask), _s(l_mask),
                                      _p(ddrop), _s(l_ddrop), _p(dbeta), _s(l_dbeta), scale), 'bs')

    def bdrln(self, inp, l_in, resid, l_resid, linear_bias, scale, bias, lin, l_lin, mask, l_mask,
              diff, l_diff, normed, l_normed, out, l_out, istd, l_istd, p=0.0, site=1):
        _lib.check(self.lib.sub_op_bdrln(
            self._pre(), _p(inp), _s(l_in), _p(resid), _s(l_resid), _p(linear_bias), _p(scale),
            _p(bias), _p(lin), _s(l_lin), _p(mask), _s(l_mask), _p(diff), _s(l_diff), _p(normed),
            _s(l_normed), _p(out), _s(l_out), _p(istd), _s(l_istd), p, site), 'bdrln')

    def blnrd(self, dout, l_dout, istd, l_istd, diff, l_diff, mask, l_mask, d_ln_in, l_d_ln_in,
              d_drop_in, l_d_drop_in):
        _lib.check(self.lib.sub_op_blnrd(
            self._pre(), _p(dout), _s(l_dout), _p(istd), _s(l_istd), _p(diff), _s(l_diff), _p(mask),
            _s(l_mask), _p(d_ln_in), _s(l_d_ln_in), _p(d_drop_in), _s(l_d_drop_in)), 'blnrd')

    def bad(self, inp, l_in, bias, lin, l_lin, mask, l_mask, out, l_out, p=0.0, site=2):
        _lib.check(self.lib.sub_op_bad(self._pre(), _p(inp), _s(l_in), _p(bias), _p(lin), _s(l_lin),
                                       _p(mask), _s(l_mask), _p(out), _s(l_out), p, site), 'bad')

    def bsb(self, inp, l_in, scale, dout, l_dout, din, l_din, dscale, dbias):
        _lib.check(self.lib.sub_op_bsb(self._pre(), _p(inp), _s(l_in), _p(scale), _p(dout), _s(l_dout),
                                       _p(din), _s(l_din), _p(dscale), _p(dbias)), 'bsb')

    def ebsb(self, inp, l_in, scale, dout1, l_dout1, dout2, l_dout2, dlinear, l_dlinear, din, l_din,
             dscale, dbias, dlinear_bias):
        _lib.check(self.lib.sub_op_ebsb(
            self._pre(), _p(inp), _s(l_in), _p(scale), _p(dout1), _s(l_dout1), _p(dout2), _s(l_dout2),
            _p(dlinear), _s(l_dlinear), _p(din), _s(l_din), _p(dscale), _p(dbias), _p(dlinear_bias)),
            'ebsb')

    def ln_backward(self, inp, l_in, scale, dout1, l_dout1, istd, l_istd, diff, l_diff, mask, l_mask, g, l_g,
                    d_ln_in, l_d_ln_in, d_drop_in, l_d_drop_in, dscale, dbias, dout2=None, l_dout2=None,
                    dlinear=None, l_dlinear=None, dlinear_bias=None, dout_bias=None, static_scratch=False):
        """bsb + blnrd, or with dout2 / dlinear / dlinear_bias / dout_bias given ebsb + blnrd + baob, in one
        launch where the sizes and layouts allow.  ``static_scratch``: the entry point that allocates
        nothing (partial sums in the library's static device array)."""
        ext = dout2 is not None
        fn = self.lib.sub_op_ln_backward_static if static_scratch else self.lib.sub_op_ln_backward
        _lib.check(fn(
            self._pre(), int(ext), _p(inp), _s(l_in), _p(scale), _p(dout1), _s(l_dout1), _p(dout2),
            _s(l_dout2 or l_dout1), _p(dlinear), _s(l_dlinear or l_dout1), _p(istd), _s(l_istd), _p(diff), _s(l_diff),
            _p(mask), _s(l_mask), _p(g), _s(l_g), _p(d_ln_in), _s(l_d_ln_in), _p(d_drop_in), _s(l_d_drop_in),
            _p(dscale), _p(dbias), _p(dlinear_bias), _p(dout_bias)), 'ln_backward')

    def bdrlb(self, ddrop, l_ddrop, mask, l_mask, lin, l_lin, dlinear, l_dlinear, dbias):
        _lib.check(self.lib.sub_op_bdrlb(self._pre(), _p(ddrop), _s(l_ddrop), _p(mask), _s(l_mask),
                                         _p(lin), _s(l_lin), _p(dlinear), _s(l_dlinear), _p(dbias)),
                   'bdrlb')

    def baob(self, datt, l_datt, dbo):
        _lib.check(self.lib.sub_op_baob(self._pre(), _p(datt), _s(l_datt), _p(dbo)), 'baob')

    def aib(self, inp, l_in, bias, l_bias, out, l_out):
        _lib.check(self.lib.sub_op_aib(self._pre(), _p(inp), _s(l_in), _p(bias), _s(l_bias), _p(out),
                                       _s(l_out)), 'aib')

    def baib(self, d, l_d, dbias, l_dbias):
        _lib.check(self.lib.sub_op_baib(self._pre(), _p(d), _s(l_d), _p(dbias), _s(l_dbias)), 'baib')

    def bei(self, dxatt, l_dxatt, dresid1, l_dresid1, dx, l_dx):
        _lib.check(self.lib.sub_op_bei(self._pre(), _p(dxatt), _s(l_dxatt), _p(dresid1),
                                       _s(l_dresid1), _p(dx), _s(l_dx)), 'bei')

    def relayout(self, src, l_src, dst, l_dst):
        """dst (order l_dst) = src (order l_src): the same tensor in another dimension order."""
        _lib.check(self.lib.sub_op_relayout(self._pre(), _p(src), _s(l_src), _p(dst), _s(l_dst)), 'relayout')

    def einsum_bad(self, a, l_a, b, l_b, bias, l_bias, lin, out, l_out, bits, p=0.0, site=2):
        """out = dropout(act(einsum(a, b) + bias)) in one launch where the product qualifies
        (then True; False: nothing was launched).  ``bits``: a uint8 tensor of numel(out) / 8
        bytes for einsum_bdrlb; ``lin`` receives the pre-activation (GELU; may be None with ReLU)."""
        applied = ctypes.c_int(0)
        _lib.check(self.lib.sub_op_einsum_bad(
            self._pre(), _p(a), _s(l_a), _p(b), _s(l_b), _p(bias), _s(l_bias), _p(lin), _p(out), _s(l_out),
            ctypes.c_void_p(bits.data_ptr()), p, site, ctypes.byref(applied)), 'einsum_bad')
        return bool(applied.value)

    def einsum_bdrlb(self, a, l_a, b, l_b, gate, l_gate, bits, dlinear, l_dlinear, dbias):
        """dlinear = act'(.) * keep * einsum(a, b) and dbias = its sum over the tokens, in one
        launch where the product qualifies (then True; False: nothing was launched).  ``gate``:
        the output of einsum_bad (ReLU) or its pre-activation (GELU); ``bits``: what it left."""
        applied = ctypes.c_int(0)
        _lib.check(self.lib.sub_op_einsum_bdrlb(
            self._pre(), _p(a), _s(l_a), _p(b), _s(l_b), _p(gate), _s(l_gate), ctypes.c_void_p(bits.data_ptr()),
            _p(dlinear), _s(l_dlinear), _p(dbias), ctypes.byref(applied)), 'einsum_bdrlb')
        return bool(applied.value)

    def einsum_pair(self, first, second):
        """Two independent contractions, in one launch where the pair qualifies (a data
        gradient and the weight gradient next to it).  ``first`` = (a, l_a, b, l_b, c, l_c)
        or with (addend, l_addend) appended; ``second`` = (a, l_a, b, l_b, c, l_c).
        Returns True when they ran as one launch."""
        a1, la1, b1, lb1, c1, lc1 = first[:6]
        t1, lt1 = (first[6], first[7]) if len(first) > 6 else (None, None)
        a2, la2, b2, lb2, c2, lc2 = second
        paired = ctypes.c_int(0)
        _lib.check(self.lib.sub_op_einsum_pair(
            self._pre(), _p(a1), _s(la1), _p(b1), _s(lb1), _p(t1), _s(lt1) if lt1 else None, _p(c1), _s(lc1), 1.0,
            _p(a2), _s(la2), _p(b2), _s(lb2), _p(c2), _s(lc2), 1.0, ctypes.byref(paired)), 'einsum_pair')
        return bool(paired.value)

    def einsum(self, a, l_a, b, l_b, c, l_c, alpha=1.0, addend=None, l_addend=None):
        """c = alpha * einsum(a, b) [+ addend, broadcast over the dims it lacks]."""
        if addend is not None:
            _lib.check(self.lib.sub_op_einsum_add(self._pre(), _p(a), _s(l_a), _p(b), _s(l_b), _p(addend),
                                                  _s(l_addend), _p(c), _s(l_c), alpha), 'einsum_add')
            return
        _lib.check(self.lib.sub_op_einsum(self._pre(), _p(a), _s(l_a), _p(b), _s(l_b), _p(c), _s(l_c),
                                          alpha), 'einsum')
