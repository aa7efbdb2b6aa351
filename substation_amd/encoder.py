"""PyTorch interface to the MI355X encoder layer.

Mirror of pytorch_module/encoder.py: same constructor, attributes, parameter
naming/shapes (one ``nn.Parameter`` per ``layouts['params']`` entry, shaped in
layout order), ``forward(X)`` and autograd backward returning ``(DX, *grads)``,
``debug`` capture.  Differences: nothing is compiled at construction (the
library is prebuilt, ``compilation_dir`` is accepted and unused), kernels run on
the caller's current stream, and keyword-only extras exist: ``activation``
('relu' as in the CUDA module, or 'gelu'), ``seed`` for the dropout masks,
``intermediate_size`` (default ``4 * embedding_size``, encoder.py:33),
``compact_attention``, ``persistent_workspace`` and ``canonical_state_dict``
(see the constructor).  ``EncoderStack`` chains several layers.
"""
import ctypes
import math

import torch

from . import _lib
from . import layouts as _lay

_SUPPORTED_DTYPES = (torch.float16,)


def causal_mask(seq_len, device='cuda', dtype=torch.float16):
    """-inf above the diagonal, 0 elsewhere (gen_attn_mask, substation/transformer.py:151-157)."""
    return torch.triu(torch.full((seq_len, seq_len), float('-inf'), dtype=dtype, device=device), diagonal=1)


class Encoder(torch.nn.Module):
    """Optimized BERT encoder layer (pytorch_module/encoder.py:19-162)."""

    def __init__(self, compilation_dir, batch_size, max_seq_len, num_heads, embedding_size,
                 layouts, torch_dtype,
                 softmax_dropout_probability, residual1_dropout_probability,
                 activation_dropout_probability, residual2_dropout_probability,
                 enable_debug=False, profiling=False, *, activation='relu', seed=0,
                 intermediate_size=None, compact_attention=False, persistent_workspace=False,
                 canonical_state_dict=False, compact_activation=False):
        """``compact_activation``: with ReLU the backward pass reads its gate off the
        dropout output, so the pre-activation LIN1 and DROP2MASK are neither written
        nor read; allocate 8 elements for each instead of B*L*4E (at B=8 L=512
        E=1024: 64 MiB less per layer call; GELU layers need LIN1 and ignore the
        request).  ``persistent_workspace``: the intermediates are allocated once and reused
        by every call instead of 37 ``torch.empty`` per iteration
        (pytorch_module/encoder.py:78-85,113-119); a forward call then overwrites
        what an earlier forward call saved for its backward pass, which backward()
        detects and refuses.  ``canonical_state_dict``: ``state_dict()`` holds every
        parameter in its canonical dimension order (``layouts.CANONICAL``) rather than
        in this module's layout, so a checkpoint loads into a module built with any
        other layouts."""
        super().__init__()
        if torch_dtype not in _SUPPORTED_DTYPES:
            raise NotImplementedError(
                f'{torch_dtype}: the MI355X kernels are fp16 storage / fp32 accumulate only')
        self.batch_size = batch_size
        self.max_seq_len = max_seq_len
        self.num_heads = num_heads
        self.embedding_size = embedding_size
        self.proj_size = self.embedding_size // self.num_heads
        self.intermediate_size = intermediate_size or self.embedding_size * 4
        self.softmax_dropout_probability = softmax_dropout_probability
        self.residual1_dropout_probability = residual1_dropout_probability
        self.activation_dropout_probability = activation_dropout_probability
        self.residual2_dropout_probability = residual2_dropout_probability
        self.torch_dtype = torch_dtype
        self.activation = activation
        self.seed = seed
        self.debug = {}  # captures intermediate tensors when enable_debug is set
        self.layouts = _lay.validate(layouts)
        self.enable_debug = enable_debug
        self.profiling = profiling
        self.compilation_dir = compilation_dir

        sizes = _lay.sizes_map(batch_size, max_seq_len, num_heads, embedding_size,
                               self.intermediate_size)
        self.sizes = sizes

        for param, layout in layouts['params']:
            sz = tuple(sizes[s] for s in layout)
            setattr(self, param, torch.nn.Parameter(torch.empty(*sz, dtype=self.torch_dtype)))
        self.params = tuple(getattr(self, k) for k, _ in layouts['params'])
        self.reset_parameters()

        config = _lib.make_config(
            batch_size, max_seq_len, num_heads, embedding_size, layouts,
            softmax_dropout_probability, residual1_dropout_probability,
            activation_dropout_probability, residual2_dropout_probability,
            activation=activation, seed=seed, intermediate_size=self.intermediate_size)
        self._handle = _lib.Handle(config)
        if profiling:
            self._handle.profile_enable(True)
        if enable_debug:
            # debug capture promises every named intermediate: keep the separate
            # aib / bei operators instead of fusing them into GEMM epilogues
            self._handle.set_option(_lib.OPT_FUSE_EPILOGUES, 0)
            self._handle.set_option(_lib.OPT_FUSE_SCORES, 0)
            self._handle.set_option(_lib.OPT_FUSE_ATTENTION, 0)
            self._handle.set_option(_lib.OPT_RELU_FROM_OUTPUT, 0)
            self._handle.set_option(_lib.OPT_PACKED_MASKS, 0)
            self._handle.set_option(_lib.OPT_SKIP_UNREAD, 0)
            self._handle.set_option(_lib.OPT_PRIVATE_LAYOUTS, 0)
        # compact_attention: when self-attention runs with the scores in registers,
        # four of the six score-sized tensors ([H,B,J,K]) are never touched and the
        # other two only hold 8 resp. K/8 bytes per score row; allocate just that
        # (at B=8 L=512 H=16: 5 MiB instead of 384 MiB per layer call).  The path is
        # then required: a later change that rules it out (option 4 = 0, a misaligned
        # tensor) makes forward() raise instead of writing through the small buffers.
        self.compact_attention = bool(compact_attention and not enable_debug
                                      and self._handle.attention_in_registers())
        if self.compact_attention:
            self._handle.set_option(_lib.OPT_FUSE_ATTENTION, _lib.FUSE_REQUIRED)
        rows = num_heads * batch_size * max_seq_len
        compact = {}
        if self.compact_attention:
            compact = {'BETA': 8, 'ATTN_DROP': 8, 'DATTN_DROP': 8, 'DBETA': 8,
                       'ALPHA': rows * 4, 'ATTN_DROP_MASK': rows * max(max_seq_len // 16, 1)}
        # compact_activation: as above for the two feed-forward tensors that the ReLU
        # path leaves untouched while option 6 is on; forward() and backward() check it.
        self.compact_activation = bool(compact_activation and not enable_debug and activation == 'relu'
                                       and self._handle.get_option(_lib.OPT_RELU_FROM_OUTPUT))
        if self.compact_activation:
            compact.update({'LIN1': 8, 'DROP2MASK': 8})
        self.persistent_workspace = bool(persistent_workspace)
        self.canonical_state_dict = bool(canonical_state_dict)
        self._workspace = {}           # 'forward_interm' / 'backward_interm' -> tensors, when persistent
        self._shared_backward = None   # set by EncoderStack: one backward workspace for all layers
        self._generation = 0
        handle = self._handle
        lib = handle.lib
        module = self
        n_fwd = 1 + len(layouts['params']) + len(layouts['forward_interm']) + 1
        n_bwd = 1 + len(layouts['params']) + len(layouts['backward_interm']) + (
            len(layouts['params']) + len(layouts['forward_interm']) + 1) + 1
        fwd_array = ctypes.c_void_p * n_fwd
        bwd_array = ctypes.c_void_p * n_bwd

        in_shape = tuple(sizes[s] for s in layouts['input'][1])
        out_shape = tuple(sizes[s] for s in layouts['output'][1])

        def _alloc(key, device):
            return [torch.empty(*((compact[name],) if name in compact else tuple(sizes[s] for s in layout)),
                                device=device, dtype=module.torch_dtype, requires_grad=False)
                    for name, layout in layouts[key]]

        def _workspace(key, device):
            if not module.persistent_workspace:
                return _alloc(key, device)
            if key == 'backward_interm' and module._shared_backward is not None:
                store = module._shared_backward
            else:
                store = module._workspace
            if key not in store or store[key][0].device != device:
                store[key] = _alloc(key, device)
            return store[key]

        class EncoderFunction(torch.autograd.Function):
            @staticmethod
            def forward(ctx, X, *weights):
                if not X.is_cuda:
                    raise RuntimeError('Encoder.forward needs a tensor on the GPU')
                if tuple(X.shape) != in_shape:
                    raise ValueError(f"X has shape {tuple(X.shape)}, the configured input layout "
                                     f"{layouts['input'][1]} needs {in_shape}")
                if module.compact_attention and not handle.attention_in_registers():
                    raise RuntimeError('this Encoder was built with compact_attention=True but the attention '
                                       'kernels that keep the scores in registers are switched off')
                module._check_compact_activation()
                dev = X.device
                X = X.contiguous()
                # same element count as X, shaped in the output's own dimension order
                Y = torch.empty(out_shape, device=dev, dtype=X.dtype)
                forward_intermediate = _workspace('forward_interm', dev)
                module._generation += 1
                ctx.generation = module._generation
                weights_c = [t.contiguous() for t in weights]
                handle.set_stream(torch.cuda.current_stream(dev).cuda_stream)
                ptrs = fwd_array(X.data_ptr(), *(t.data_ptr() for t in weights_c),
                                 *(t.data_ptr() for t in forward_intermediate), Y.data_ptr())
                _lib.check(lib.sub_encoder_forward(handle.ptr, ptrs, n_fwd), 'encoder_forward')
                ctx.save_for_backward(*weights_c, *forward_intermediate, X)

                if module.enable_debug:
                    torch.cuda.synchronize()
                    for idx, (name, _) in enumerate(layouts['forward_interm']):
                        module.debug[name] = forward_intermediate[idx].detach().cpu().numpy()
                    for idx, (name, _) in enumerate(layouts['params']):
                        module.debug[name] = weights[idx].detach().cpu().numpy()
                return Y

            @staticmethod
            def backward(ctx, DY):
                if module.persistent_workspace and ctx.generation != module._generation:
                    raise RuntimeError('persistent_workspace: forward() ran again before this backward pass; '
                                       'what it had saved has been overwritten')
                module._check_compact_activation()
                dev = DY.device
                DY = DY.contiguous()
                DX = torch.empty(in_shape, device=dev, dtype=DY.dtype)
                backward_intermediate = _workspace('backward_interm', dev)
                param_gradients = _alloc('params', dev)
                handle.set_stream(torch.cuda.current_stream(dev).cuda_stream)
                ptrs = bwd_array(DY.data_ptr(), *(t.data_ptr() for t in param_gradients),
                                 *(t.data_ptr() for t in backward_intermediate),
                                 *(t.data_ptr() for t in ctx.saved_tensors), DX.data_ptr())
                _lib.check(lib.sub_encoder_backward(handle.ptr, ptrs, n_bwd), 'encoder_backward')

                if module.enable_debug:
                    torch.cuda.synchronize()
                    for idx, (name, _) in enumerate(layouts['backward_interm']):
                        module.debug[name] = backward_intermediate[idx].detach().cpu().numpy()
                    for idx, (name, _) in enumerate(layouts['params']):
                        module.debug['D' + name] = param_gradients[idx].detach().cpu().numpy()
                return (DX, *param_gradients)

        self.encoder_func = EncoderFunction

    def _check_compact_activation(self):
        if self.compact_activation and not self._handle.get_option(_lib.OPT_RELU_FROM_OUTPUT):
            raise RuntimeError('this Encoder was built with compact_activation=True but the ReLU gate from '
                               'the dropout output (option 6) is switched off: LIN1 and DROP2MASK would be '
                               'written through 8-element buffers')

    def _canonical_perm(self, name, layout):
        canon = _lay.CANONICAL[name]
        return [layout.index(d) for d in canon]

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        if not self.canonical_state_dict:
            return
        for name, layout in self.layouts['params']:
            t = destination[prefix + name]
            destination[prefix + name] = t.detach().permute(self._canonical_perm(name, layout)).contiguous()

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys,
                              unexpected_keys, error_msgs):
        if self.canonical_state_dict:
            for name, layout in self.layouts['params']:
                key = prefix + name
                if key in state_dict:
                    canon = _lay.CANONICAL[name]
                    t = state_dict[key]
                    if t.dim() == len(canon):
                        state_dict[key] = t.permute([canon.index(d) for d in layout]).contiguous()
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys,
                                      unexpected_keys, error_msgs)

    def reset_parameters(self):
        """U(-1/sqrt(2), 1/sqrt(2)) for every parameter, pytorch_module/encoder.py:144-158."""
        stdev = 1.0 / math.sqrt(2)
        for weight in self.parameters():
            t = torch.empty_like(weight, dtype=torch.float32)
            torch.nn.init.uniform_(t, -stdev, stdev)
            with torch.no_grad():
                weight[:] = t

    def set_rng(self, seed, step=0):
        """Dropout masks are a pure function of (seed, site, step, element index);
        every forward call advances ``step`` by one."""
        self.seed = seed
        self._handle.set_rng(seed, step)

    def set_attention_mask(self, mask, layout='JK'):
        """Masked self-attention (the ``decoder`` layer of
        substation/transformer.py:443-546): ``mask`` is an additive [L, L] fp16 CUDA
        tensor over (query, key) positions, e.g. ``causal_mask(L)``; ``None``
        clears it.  It is added to the raw scores, before the 1/sqrt(P) scaling
        (substation/attention.py:65-68)."""
        if mask is None:
            self._attn_mask = None
            self._handle.set_attention_mask(0)
            return
        L = self.max_seq_len
        if not (mask.is_cuda and mask.dtype == self.torch_dtype and tuple(mask.shape) == (L, L)
                and mask.is_contiguous()):
            raise ValueError(f'the attention mask is a contiguous [{L}, {L}] fp16 CUDA tensor')
        self._attn_mask = mask                 # keeps the memory alive
        self._handle.set_attention_mask(mask.data_ptr(), layout)

    def use_device_step(self, counter=None):
        """Keeps the dropout step in device memory (a one-element int32 CUDA tensor,
        created at zero when not given) so that forward calls recorded in a HIP
        graph draw new masks on every replay: the step a kernel uses is the host
        step of ``set_rng`` plus this counter, which every forward advances on
        the stream.  Returns the tensor; ``use_device_step(False)`` switches back."""
        if counter is False:
            self._step_counter = None
            self._handle.set_rng_counter(0)
            return None
        if counter is None:
            counter = torch.zeros(1, dtype=torch.int32, device='cuda')
        if not (counter.is_cuda and counter.dtype == torch.int32 and counter.numel() == 1):
            raise ValueError('the step counter is a one-element int32 CUDA tensor')
        self._step_counter = counter          # keeps the memory alive
        self._handle.set_rng_counter(counter.data_ptr())
        return counter

    def profile(self):
        """Per-launch times in ms of the last forward call and, once it has been
        issued, of the backward call after it (``profiling=True`` only); the
        counterpart of the NVTX ranges of pytorch_module/encoder.cu:32-53."""
        return self._handle.profile_read()

    def forward(self, X):
        """Run the encoder.  X is in ``layouts['input'][1]`` order; the result is
        in ``layouts['output'][1]`` order."""
        return self.encoder_func.apply(X, *self.params)


class EncoderStack(torch.nn.Module):
    """``num_layers`` encoder layers applied one after the other.

    What chaining needs beyond the single layer of pytorch_module/encoder.py: the
    output layout must equal the input layout (config_selection/ops.py:265-270
    ties them for this reason; checked here), every layer draws its dropout masks
    from its own stream (seed + layer index), the forward intermediates of each
    layer are allocated once and reused by every iteration, all layers share one
    set of backward intermediates (only one layer's backward pass is running at a
    time), and ``state_dict()`` is in canonical dimension order so that a
    checkpoint does not depend on the layouts the stack was built with."""

    def __init__(self, num_layers, batch_size, max_seq_len, num_heads, embedding_size, layouts, torch_dtype,
                 softmax_dropout_probability, residual1_dropout_probability,
                 activation_dropout_probability, residual2_dropout_probability, *, activation='relu', seed=0,
                 intermediate_size=None, compact_attention=True, persistent_workspace=True,
                 canonical_state_dict=True, profiling=False, compact_activation=True):
        super().__init__()
        if layouts['input'][1] != layouts['output'][1]:
            raise ValueError(f"layers stack only when the output layout ({layouts['output'][1]}) equals the "
                             f"input layout ({layouts['input'][1]})")
        self.num_layers = num_layers
        self.layers = torch.nn.ModuleList([
            Encoder('unused', batch_size, max_seq_len, num_heads, embedding_size, layouts, torch_dtype,
                    softmax_dropout_probability, residual1_dropout_probability,
                    activation_dropout_probability, residual2_dropout_probability, profiling=profiling,
                    activation=activation, seed=seed + i, intermediate_size=intermediate_size,
                    compact_attention=compact_attention, persistent_workspace=persistent_workspace,
                    canonical_state_dict=canonical_state_dict, compact_activation=compact_activation)
            for i in range(num_layers)])
        shared = {}
        for layer in self.layers:
            layer._shared_backward = shared

    def forward(self, X):
        for layer in self.layers:
            X = layer(X)
        return X

    def set_rng(self, seed, step=0):
        """Layer i draws from the stream of ``seed + i``."""
        for i, layer in enumerate(self.layers):
            layer.set_rng(seed + i, step)

    def set_attention_mask(self, mask, layout='JK'):
        for layer in self.layers:
            layer.set_attention_mask(mask, layout)

    def workspace_bytes(self):
        """Device bytes held by the persistent workspaces (0 before the first call)."""
        seen, total = set(), 0
        stores = [layer._workspace for layer in self.layers]
        stores += [layer._shared_backward for layer in self.layers if layer._shared_backward is not None]
        for store in stores:
            if id(store) in seen:
                continue
            seen.add(id(store))
            total += sum(t.numel() * t.element_size() for ts in store.values() for t in ts)
        return total
