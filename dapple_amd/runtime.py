"""The explicit per-stage runtime the reference only implies with graph edges.

``schedule_ops`` states the early-backward rule of bert/graph.py:126-132 (and the
``2S-1`` variant of vgg19/tf-keras-dapple.py:292) as the op order of one stage;
``StageRuntime.step`` issues ``ds_stage_forward`` / ``ds_stage_backward`` in that
order with a stash of K = S - i slots, and the weight gradients accumulate in
place in one flat fp32 buffer (bert/graph.py:145-161: a sum over micro-batches).
"""
import ctypes as C

import torch

from . import _lib
from ._lib import DS_BF16, DS_F32, DS_STAGE_BERT, GnmtCfg, StageCfg, VggCfg, XlnetCfg, check, ptr


def stash_depth(stage_index, num_stages, variant="S"):
    """In-flight micro-batches at a stage: S - i (bert/graph.py:129) or 2S - 1 - i (vgg19/tf-keras-dapple.py:292)."""
    if variant not in ("S", "2S-1"):
        raise ValueError("variant must be 'S' or '2S-1'")
    return (num_stages if variant == "S" else 2 * num_stages - 1) - stage_index


def schedule_ops(stage_index, num_stages, num_micro_batches, variant="S"):
    """[('F', j) | ('B', j)] in execution order: K warm-up forwards, then one backward per forward.  K is the number of
    forwards the reference's control edges let a stage run ahead (bert/graph.py:126-132: S - i; vgg19/tf-keras-dapple.py:292:
    2S - 1 - i).  For the first stage this is the order the graph executes in; under the "2S-1" rule a later stage's
    backward is ready earlier than that, so there the list is the deepest order the edges allow (and what the stash is
    sized for), one of several valid executions with identical results."""
    if not (0 <= stage_index < num_stages):
        raise ValueError("stage_index %d outside [0, %d)" % (stage_index, num_stages))
    if num_micro_batches < 1:
        raise ValueError("num_micro_batches must be >= 1")
    k = min(stash_depth(stage_index, num_stages, variant), num_micro_batches)
    ops = [("F", j) for j in range(k)]
    for j in range(num_micro_batches):
        ops.append(("B", j))
        if j + k < num_micro_batches:
            ops.append(("F", j + k))
    return ops


_TORCH_DTYPE = {DS_F32: torch.float32, DS_BF16: torch.bfloat16}


class Stage:
    """Owns a ``ds_stage`` handle plus the flat fp32 master weights / gradients it is bound to."""

    def __init__(self, handle, act_dtype, in_numel, out_numel, stash_slots, in_dtype=None, takes_input_grad=True,
                 device="cuda:0", cfg=None):
        self.lib = _lib.load()
        self.device = torch.device(device)
        self._h = handle
        self.cfg = cfg
        self.act_dtype = act_dtype
        self.in_dtype = act_dtype if in_dtype is None else in_dtype
        self.in_numel, self.out_numel = in_numel, out_numel
        self.stash_slots = stash_slots
        self.takes_input_grad = takes_input_grad
        self.with_embedding = not takes_input_grad
        n = self.lib.ds_stage_num_weights(self._h)
        self.weight_names, self.weight_shapes = [], []
        buf = C.create_string_buffer(256)
        numel, rows, cols = C.c_int64(), C.c_int64(), C.c_int64()
        for i in range(n):
            check(self.lib.ds_stage_weight_info(self._h, i, buf, 256, C.byref(numel), C.byref(rows), C.byref(cols)),
                  "ds_stage_weight_info")
            name = buf.value.decode()
            self.weight_names.append(name)
            vector = name.endswith(("/bias", "/gamma", "/beta"))
            self.weight_shapes.append((cols.value,) if vector else (rows.value, cols.value))
        self.weights, self.grads = {}, {}
        self.flat_weights = self.flat_grads = None
        self._weights_stale = False
        self.overlap = False

    # -- weights ---------------------------------------------------------------------------
    def bind(self, weights):
        """weights: {reference variable name: array/tensor}. Copies into one flat fp32 buffer,
        allocates the flat master-gradient buffer (zeroed) and binds both.  A weight may come in the
        reference's own shape (e.g. an HWIO conv kernel) as long as its element count matches."""
        missing = [n for n in self.weight_names if n not in weights]
        if missing:
            raise KeyError("missing weights: %s" % missing[:4])
        sizes, shapes = [], []
        for n, shp in zip(self.weight_names, self.weight_shapes):
            numel = 1
            for s in shp:
                numel *= s
            w = weights[n]
            wn = 1
            for s in tuple(w.shape):
                wn *= s
            if wn != numel:
                raise ValueError("weight %s has shape %s, stage expects %s" % (n, tuple(w.shape), tuple(shp)))
            shapes.append(tuple(w.shape))
            sizes.append((numel + 63) // 64 * 64)          # keep every view 256-byte aligned
        total = sum(sizes)
        self.flat_weights = torch.empty(total, dtype=torch.float32, device=self.device)
        self.flat_grads = torch.zeros(total, dtype=torch.float32, device=self.device)
        off = 0
        self.weight_offsets, self.weight_numels = [], []
        wp = (C.c_void_p * len(sizes))()
        gp = (C.c_void_p * len(sizes))()
        for i, (n, shp, sz) in enumerate(zip(self.weight_names, shapes, sizes)):
            numel = 1
            for s in shp:
                numel *= s
            wv = self.flat_weights[off:off + numel].view(*shp)
            wv.copy_(torch.as_tensor(weights[n], dtype=torch.float32))
            self.weights[n] = wv
            self.grads[n] = self.flat_grads[off:off + numel].view(*shp)
            wp[i], gp[i] = wv.data_ptr(), self.grads[n].data_ptr()
            self.weight_offsets.append(off)
            self.weight_numels.append(numel)
            off += sz
        check(self.lib.ds_stage_bind_weights(self._h, len(sizes), wp, gp), "ds_stage_bind_weights")

    def refresh_weights(self):
        check(self.lib.ds_stage_refresh_weights(self._h), "ds_stage_refresh_weights")
        self._weights_stale = False

    def mark_weights_stale(self):
        """The master weights changed (an optimizer step): the next forward pass rebuilds the compute copies first."""
        self._weights_stale = True

    def zero_grads(self):
        self.flat_grads.zero_()

    # -- one micro-batch ---------------------------------------------------------------------
    def _check_tensor(self, t, what, dtype, numel):
        """The kernels take raw device pointers: anything but a contiguous tensor on this stage's GPU would fault there."""
        if not t.is_cuda or t.device != torch.device(self.device):
            raise ValueError("%s must live on %s (got %s)" % (what, self.device, t.device))
        if not t.is_contiguous():
            raise ValueError("%s must be contiguous" % what)
        if t.dtype != dtype or t.numel() != numel:
            raise ValueError("%s must be %s with %d elements" % (what, dtype, numel))

    def forward(self, slot, x, out, key_mask=None, token_type_ids=None):
        self._check_tensor(x, "stage input", self.in_dtype, self.in_numel)
        self._check_tensor(out, "stage output", self.act_dtype, self.out_numel)
        if self._weights_stale:
            self.refresh_weights()
        if token_type_ids is not None:
            self._check_tensor(token_type_ids, "token_type_ids", torch.int32, self.in_numel)
            check(self.lib.ds_stage_set_token_types(self._h, slot, ptr(token_type_ids)), "ds_stage_set_token_types")
        if key_mask is not None:
            if key_mask.dtype != torch.float32 or not key_mask.is_cuda or not key_mask.is_contiguous():
                raise ValueError("key_mask must be a contiguous fp32 [batch, seq] tensor on the GPU")
        check(self.lib.ds_stage_forward(self._h, slot, ptr(x), ptr(key_mask), ptr(out)), "ds_stage_forward")

    def backward(self, slot, d_out, d_in=None, ready=False):
        """``ready``: when the upstream gradient may be read.  False (default): after everything queued so far on the
        stage's stream.  None: it is already complete (synthetic, or produced before this micro-batch's forward pass).
        A ``torch.cuda.Event`` or a raw event handle (``Stage.backward_event`` of the next stage): after that event -
        with forward/backward overlap on, the last two keep an earlier-queued forward pass running beside this pass."""
        self._check_tensor(d_out, "upstream gradient", self.act_dtype, self.out_numel)
        if d_in is not None:
            self._check_tensor(d_in, "input gradient", self.act_dtype, self.in_numel)
        if ready is False:
            check(self.lib.ds_stage_backward(self._h, slot, ptr(d_out), ptr(d_in)), "ds_stage_backward")
            return
        if isinstance(ready, torch.cuda.Event):
            ready = ready.cuda_event
        ev = C.c_void_p(ready) if ready is not None else None
        check(self.lib.ds_stage_backward_after(self._h, slot, ptr(d_out), ptr(d_in), ev), "ds_stage_backward_after")

    def forward_backward(self, fslot, x, out, bslot, d_out, d_in=None, key_mask=None):
        """F(fslot) and B(bslot) of two different micro-batches as one call (``ds_stage_forward_backward``): stages that
        pair passes walk both chains together, one launch per level; the others run the two passes one after the other.
        The upstream gradient must already be ordered on the current stream."""
        self._check_tensor(x, "stage input", self.in_dtype, self.in_numel)
        self._check_tensor(out, "stage output", self.act_dtype, self.out_numel)
        self._check_tensor(d_out, "upstream gradient", self.act_dtype, self.out_numel)
        if d_in is not None:
            self._check_tensor(d_in, "input gradient", self.act_dtype, self.in_numel)
        if key_mask is not None:
            if key_mask.dtype != torch.float32 or not key_mask.is_cuda or not key_mask.is_contiguous():
                raise ValueError("key_mask must be a contiguous fp32 [batch, seq] tensor on the GPU")
        if self._weights_stale:
            self.refresh_weights()
        check(self.lib.ds_stage_forward_backward(self._h, fslot, ptr(x), ptr(key_mask), ptr(out), bslot, ptr(d_out), ptr(d_in)),
              "ds_stage_forward_backward")

    def release(self, slot):
        """Gives up the micro-batch forwarded into ``slot`` without a backward pass (forward-only use)."""
        check(self.lib.ds_stage_release_slot(self._h, slot), "ds_stage_release_slot")

    def backward_event(self, slot):
        """Raw handle of the event that completes when the last backward pass of ``slot`` has written its input gradient
        (None on one stream: the pass is ordered on the stage's stream)."""
        return self.lib.ds_stage_backward_event(self._h, slot)

    def wait_backward(self, slot, stream=None):
        """Puts ``stream`` (default: the current one) behind the last backward pass of ``slot``."""
        s = _lib.current_stream() if stream is None else C.c_void_p(stream.cuda_stream)
        check(self.lib.ds_stage_wait_backward(self._h, slot, s), "ds_stage_wait_backward")

    def sync(self):
        check(self.lib.ds_stage_sync(self._h), "ds_stage_sync")

    # -- forward/backward overlap (backward passes on a second stream of the handle) --------------
    def overlap_supported(self):
        return bool(self.lib.ds_stage_overlap_supported(self._h))

    def enable_overlap(self, on=True):
        check(self.lib.ds_stage_enable_overlap(self._h, 1 if on else 0), "ds_stage_enable_overlap")
        self.overlap = bool(on)

    def join(self):
        """Orders queued backward work before whatever is queued next on the stage's stream."""
        check(self.lib.ds_stage_join(self._h), "ds_stage_join")

    def workspace_bytes(self):
        return self.lib.ds_stage_workspace_bytes(self._h)

    def stash_bytes(self, slots=None):
        return self.lib.ds_stage_stash_bytes(self._h, self.stash_slots if slots is None else slots)

    def close(self):
        if self._h:
            self.lib.ds_stage_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _dtype_code(dtype):
    return {"fp32": DS_F32, "bf16": DS_BF16, DS_F32: DS_F32, DS_BF16: DS_BF16}[dtype]


def bert_stage(num_layers, hidden, heads, ffn, batch, seq, dtype, stash_slots, embeddings=None, first_layer=0,
               ln_eps=1e-12, device="cuda:0", wgrad_group=1, residual_fp32=True):
    """A BERT stage: ``num_layers`` encoder layers, behind the embedding when ``embeddings`` =
    (vocab, type_vocab, max_pos) is given.  ``wgrad_group`` = G > 1: the weight gradients of G consecutive
    backward passes are formed by one GEMM per weight (G more stash positions; the gradients are complete
    after ``Stage.join`` / ``Stage.sync``).  ``residual_fp32`` (bf16 stages): keep the residual stream in fp32 and round
    to bf16 only the GEMM / attention operands, as the reference's fp32 graph does for the stream."""
    if hidden % heads != 0:
        raise ValueError("The hidden size (%d) is not a multiple of the number of attention heads (%d)" % (hidden, heads))
    lib = _lib.load()
    cfg = StageCfg()
    cfg.kind, cfg.dtype, cfg.num_layers = DS_STAGE_BERT, _dtype_code(dtype), num_layers
    cfg.hidden, cfg.heads, cfg.ffn, cfg.batch, cfg.seq = hidden, heads, ffn, batch, seq
    if embeddings is not None:
        cfg.with_embedding = 1
        cfg.vocab, cfg.type_vocab, cfg.max_pos = embeddings
    cfg.ln_eps, cfg.stash_slots, cfg.first_layer = ln_eps, stash_slots, first_layer
    cfg.wgrad_group = int(wgrad_group)
    cfg.residual_fp32 = 1 if residual_fp32 else 0
    h = C.c_void_p()
    with torch.cuda.device(torch.device(device)):
        check(lib.ds_stage_create(C.byref(cfg), _lib.current_stream(), C.byref(h)), "ds_stage_create")
    act = _TORCH_DTYPE[cfg.dtype]
    rows = batch * seq
    if embeddings is not None:
        return Stage(h, act, rows, rows * hidden, stash_slots, in_dtype=torch.int32, takes_input_grad=False,
                     device=device, cfg=cfg)
    return Stage(h, act, rows * hidden, rows * hidden, stash_slots, device=device, cfg=cfg)


def vgg_stage(layers, batch, height, width, in_channels, stash_slots, need_input_grad=False, dtype="fp32",
              device="cuda:0"):
    """A VGG19 conv stack: ``layers`` = [(name, out_channels | None for a 2x2 max-pool), ...] in the
    order vgg19/applications/vgg19_slice_model.py:280-302 applies them."""
    lib = _lib.load()
    cfg = VggCfg()
    cfg.dtype = _dtype_code(dtype)
    cfg.batch, cfg.height, cfg.width, cfg.in_channels = batch, height, width, in_channels
    if len(layers) > 40:
        raise ValueError("at most 40 ops")
    cfg.num_ops = len(layers)
    h_, w_, c_ = height, width, in_channels
    for i, (_, cout) in enumerate(layers):
        cfg.ops[i] = 0 if cout is None else cout
        if cout is None:
            h_, w_ = h_ // 2, w_ // 2
        else:
            c_ = cout
    cfg.stash_slots, cfg.need_input_grad = stash_slots, 1 if need_input_grad else 0
    h = C.c_void_p()
    with torch.cuda.device(torch.device(device)):
        check(lib.ds_vgg_stage_create(C.byref(cfg), _lib.current_stream(), C.byref(h)), "ds_vgg_stage_create")
    st = VggStage(h, _TORCH_DTYPE[cfg.dtype], batch * height * width * in_channels, batch * h_ * w_ * c_, stash_slots,
                  takes_input_grad=need_input_grad, device=device, cfg=cfg)
    st.out_shape = (batch, h_, w_, c_)
    # the handle numbers its convs block%d_conv%d from block 1; a stage that starts further down the model (the last
    # device: block5_conv3 ...) goes by the caller's layer names, which are the reference's variable scopes
    st.layer_names = [n for n, c in layers if c is not None]
    if len(st.weight_names) == 2 * len(st.layer_names):
        st.weight_names = [n + sfx for n in st.layer_names for sfx in ("/kernel", "/bias")]
    return st


def gnmt_stage(num_layers, units, vocab, batch, seq, stash_slots, forget_bias=1.0, dtype="fp32", device="cuda:0"):
    """The GNMT encoder stage (gnmt/nmt/gnmt_model.py:61-221): ids [batch, seq] int32 -> [seq, batch, units]."""
    lib = _lib.load()
    cfg = GnmtCfg()
    cfg.dtype, cfg.num_layers, cfg.units, cfg.vocab = _dtype_code(dtype), num_layers, units, vocab
    cfg.batch, cfg.seq, cfg.forget_bias, cfg.stash_slots = batch, seq, forget_bias, stash_slots
    h = C.c_void_p()
    with torch.cuda.device(torch.device(device)):
        check(lib.ds_gnmt_stage_create(C.byref(cfg), _lib.current_stream(), C.byref(h)), "ds_gnmt_stage_create")
    st = GnmtStage(h, _TORCH_DTYPE[cfg.dtype], batch * seq, seq * batch * units, stash_slots, in_dtype=torch.int32,
                   takes_input_grad=False, device=device, cfg=cfg)
    st.out_shape = (seq, batch, units)
    return st


def gnmt_decoder_stage(num_layers, units, batch, seq, stash_slots, first_layer=1, forget_bias=1.0, dtype="fp32", device="cuda:0"):
    """Decoder cells ``first_layer .. first_layer + num_layers - 1`` as the reference's second device runs them
    (GNMTAttentionMultiCell_2, gnmt/nmt/gnmt_model.py:489-537; model.py:641-656): [seq, batch, units] -> [seq, batch, units]."""
    lib = _lib.load()
    cfg = GnmtCfg()
    cfg.dtype, cfg.num_layers, cfg.units, cfg.vocab = _dtype_code(dtype), num_layers, units, 0
    cfg.batch, cfg.seq, cfg.forget_bias, cfg.stash_slots = batch, seq, forget_bias, stash_slots
    cfg.part, cfg.first_layer = 1, first_layer
    h = C.c_void_p()
    with torch.cuda.device(torch.device(device)):
        check(lib.ds_gnmt_stage_create(C.byref(cfg), _lib.current_stream(), C.byref(h)), "ds_gnmt_stage_create")
    n = seq * batch * units
    st = GnmtStage(h, _TORCH_DTYPE[cfg.dtype], n, n, stash_slots, device=device, cfg=cfg)
    st.out_shape = (seq, batch, units)
    return st


def gnmt_attention_stage(units, vocab, batch, seq, src_seq, stash_slots, forget_bias=1.0, dtype="fp32", device="cuda:0"):
    """Decoder cell 0 under the attention wrapper, on the first device behind the encoder (gnmt/nmt/gnmt_model.py:309-325,
    :366-374, :440-487; model.py:622-640): memory [src_seq, batch, units] -> cell outputs [seq, batch, units]."""
    lib = _lib.load()
    cfg = GnmtCfg()
    cfg.dtype, cfg.num_layers, cfg.units, cfg.vocab = _dtype_code(dtype), 1, units, vocab
    cfg.batch, cfg.seq, cfg.forget_bias, cfg.stash_slots = batch, seq, forget_bias, stash_slots
    cfg.part, cfg.src_seq = 2, src_seq
    h = C.c_void_p()
    with torch.cuda.device(torch.device(device)):
        check(lib.ds_gnmt_stage_create(C.byref(cfg), _lib.current_stream(), C.byref(h)), "ds_gnmt_stage_create")
    st = GnmtStage(h, _TORCH_DTYPE[cfg.dtype], src_seq * batch * units, seq * batch * units, stash_slots, device=device, cfg=cfg)
    st.out_shape = (seq, batch, units)
    return st


class VggStage(Stage):
    def read_activation(self, slot, op, shape):
        """The stashed output of op ``op`` (NHWC fp32, ``shape``) of the micro-batch forwarded into ``slot``."""
        t = torch.empty(shape, dtype=torch.float32, device=self.device)
        check(self.lib.ds_vgg_stage_read_activation(self._h, slot, op, ptr(t), t.numel()), "ds_vgg_stage_read_activation")
        return t


class GnmtStage(Stage):
    def set_decoder_inputs(self, slot, target_input, source_sequence_length=None, attention_out=None):
        """Attention-cell stage: side inputs of the micro-batch about to be forwarded into ``slot``: target_input int32
        [batch, seq], source_sequence_length int32 [batch] (None: full length), attention_out fp32 [seq, batch, units] that the
        forward pass fills with every step's attention vector (keep it alive until then)."""
        b, t = self.cfg.batch, self.cfg.seq
        if target_input.dtype != torch.int32 or not target_input.is_cuda or not target_input.is_contiguous() or target_input.numel() != b * t:
            raise ValueError("target_input must be a contiguous int32 GPU tensor of [batch, seq]")
        if source_sequence_length is not None and (source_sequence_length.dtype != torch.int32 or not source_sequence_length.is_cuda
                                                   or source_sequence_length.numel() != b):
            raise ValueError("source_sequence_length must be an int32 GPU tensor of [batch]")
        if attention_out is not None and (attention_out.dtype != torch.float32 or not attention_out.is_cuda or not attention_out.is_contiguous()
                                          or attention_out.numel() != self.out_numel):
            raise ValueError("attention_out must be a contiguous fp32 GPU tensor of [seq, batch, units]")
        check(self.lib.ds_gnmt_stage_set_decoder_inputs(self._h, slot, ptr(target_input), ptr(source_sequence_length), ptr(attention_out)),
              "ds_gnmt_stage_set_decoder_inputs")

    def set_attention(self, slot, attention=None):
        """Decoder stage: the attention vectors [seq, batch, units] fp32 every cell of the micro-batch about to be
        forwarded into ``slot`` concatenates to its input (None: zeros).  No gradient flows into them."""
        if attention is not None and (attention.dtype != torch.float32 or not attention.is_cuda or not attention.is_contiguous()
                                      or attention.numel() != self.out_numel):
            raise ValueError("attention must be a contiguous fp32 GPU tensor of [seq, batch, units]")
        check(self.lib.ds_gnmt_stage_set_attention(self._h, slot, ptr(attention)), "ds_gnmt_stage_set_attention")

    def set_lengths(self, slot, lengths=None):
        """``source_sequence_length`` [batch] int32 of the micro-batch about to be forwarded into ``slot``
        (None: full length)."""
        if lengths is not None and (lengths.dtype != torch.int32 or not lengths.is_cuda or not lengths.is_contiguous()
                                    or lengths.numel() != self.cfg.batch):
            raise ValueError("lengths must be a contiguous int32 GPU tensor of [batch]")
        check(self.lib.ds_gnmt_stage_set_lengths(self._h, slot, ptr(lengths)), "ds_gnmt_stage_set_lengths")


class XlnetStage(Stage):
    def set_inputs(self, slot, masks=None, seg_mat=None, mems=None):
        """Side inputs of the micro-batch about to be forwarded into ``slot``: masks fp32
        [streams, seq, klen, batch] (1 = masked), seg_mat uint8 [seq, klen, batch], mems [layers, mem_len, batch, hidden]."""
        for t, dt in ((masks, torch.float32), (seg_mat, torch.uint8), (mems, self.act_dtype)):
            if t is not None and (t.dtype != dt or not t.is_cuda or not t.is_contiguous()):
                raise ValueError("side input must be a contiguous GPU tensor of %s" % dt)
        check(self.lib.ds_xlnet_stage_set_inputs(self._h, slot, ptr(masks), ptr(seg_mat), ptr(mems)), "ds_xlnet_stage_set_inputs")


def xlnet_stage(num_layers, hidden, heads, ffn, batch, seq, dtype, stash_slots, mem_len=0, streams=1, first_layer=0,
                ln_eps=1e-14, device="cuda:0", attention="auto", residual_fp32=True, wgrad_group=1):
    """An XLNet stage of ``num_layers`` relative-attention layers (xlnet/models/slice_xlnet.py:164-180).
    ``attention`` (``ds_xlnet_cfg.fused_attention``): "auto" = scores, relative shift and softmax as one kernel per pass where
    the shape allows; "separate" = every product and the softmax as launches of their own.  ``residual_fp32`` (bf16 stages): keep the
    residual stream in fp32 (``ds_xlnet_cfg.residual_fp32``).  ``wgrad_group`` = G > 1 (bf16): weight gradients once per G
    backward passes, one product per weight over all G micro-batches; call ``set_inputs`` before every forward pass then."""
    lib = _lib.load()
    cfg = XlnetCfg()
    cfg.dtype, cfg.num_layers, cfg.hidden, cfg.heads, cfg.ffn = _dtype_code(dtype), num_layers, hidden, heads, ffn
    cfg.batch, cfg.seq, cfg.mem_len, cfg.streams = batch, seq, mem_len, streams
    cfg.ln_eps, cfg.first_layer, cfg.stash_slots = ln_eps, first_layer, stash_slots
    modes = {"auto": 0, "separate": 1}
    if attention not in modes:
        raise ValueError("attention must be one of %r" % (list(modes),))
    cfg.fused_attention = modes[attention]
    cfg.residual_fp32 = 1 if residual_fp32 else 0
    cfg.wgrad_group = wgrad_group
    h = C.c_void_p()
    with torch.cuda.device(torch.device(device)):
        check(lib.ds_xlnet_stage_create(C.byref(cfg), _lib.current_stream(), C.byref(h)), "ds_xlnet_stage_create")
    n = streams * seq * batch * hidden
    st = XlnetStage(h, _TORCH_DTYPE[cfg.dtype], n, n, stash_slots, device=device, cfg=cfg)
    st.out_shape = (streams, seq, batch, hidden)
    return st


class StageRuntime:
    """Runs one stage over M micro-batches in the early-backward order."""

    def __init__(self, stage, stage_index=0, num_stages=2, num_micro_batches=8, variant="S", needs_input_grad=True,
                 pair_passes=False):
        """``pair_passes``: where the order has F(j+1) directly in front of B(j) - its steady state - issue the two as one
        ``Stage.forward_backward`` call (same results; stages that pair passes run them level by level in one launch each)."""
        self.stage = stage
        self.pair_passes = bool(pair_passes)
        self.ops = schedule_ops(stage_index, num_stages, num_micro_batches, variant)
        self.k = min(stash_depth(stage_index, num_stages, variant), num_micro_batches)
        if stage.stash_slots < self.k:
            raise ValueError("stage has %d stash slots, the schedule needs %d" % (stage.stash_slots, self.k))
        self.m = num_micro_batches
        self.needs_input_grad = needs_input_grad and stage.takes_input_grad

    def step(self, inputs, upstream, outputs, input_grads=None, key_masks=None, before_forward=None):
        """inputs[M], upstream[M]: device tensors; outputs[M] (and input_grads[M]) are filled.
        Weight gradients add into ``stage.grads`` (call ``stage.zero_grads()`` between steps)."""
        if len(inputs) != self.m or len(upstream) != self.m or len(outputs) != self.m:
            raise ValueError("expected %d micro-batches" % self.m)
        slot_of, free = {}, list(range(self.stage.stash_slots))
        # the upstream gradients exist when the step starts: with forward/backward overlap a backward pass waits for
        # this point of the current stream, not for the forward passes queued after it
        ready = None
        if self.stage.overlap:
            ready = torch.cuda.Event()
            ready.record()
        i = 0
        while i < len(self.ops):
            op, j = self.ops[i]
            i += 1
            if op == "F":
                slot = free.pop(0)
                slot_of[j] = slot
                if before_forward is not None:
                    before_forward(slot, j)          # e.g. XlnetStage.set_inputs for this micro-batch
                mask = None if key_masks is None else key_masks[j]
                if self.pair_passes and i < len(self.ops) and self.ops[i][0] == "B":
                    jb = self.ops[i][1]
                    i += 1
                    bslot = slot_of.pop(jb)
                    d_in = input_grads[jb] if (self.needs_input_grad and input_grads is not None) else None
                    self.stage.forward_backward(slot, inputs[j], outputs[j], bslot, upstream[jb], d_in, key_mask=mask)
                    free.append(bslot)
                    continue
                self.stage.forward(slot, inputs[j], outputs[j], mask)
            else:
                slot = slot_of.pop(j)
                d_in = input_grads[j] if (self.needs_input_grad and input_grads is not None) else None
                self.stage.backward(slot, upstream[j], d_in, ready=ready)
                free.append(slot)
        self.stage.join()
        return outputs


class PipelineRuntime:
    """All S stages of a sliced model on ONE GPU, M micro-batches: the unrolled graph of bert/graph.py:97-161 with the
    stage boundaries as device tensors instead of sends.  Every stage issues its own early-backward order
    (``schedule_ops(i, S, M)``, the rule of bert/graph.py:126-132); an operation is issued once its data is there -
    F(i, j) after F(i-1, j), B(i, j) after B(i+1, j), the last stage's backward after ``loss_fn`` - so the global order
    is one the reference's control dependencies allow.  ``loss_fn(j, last_output) -> (loss, d_last_output)`` is the
    last stage's head.  Stages with forward/backward overlap on run their backward passes on streams of their own: the
    gradient a stage hands down then travels with the event of the pass that wrote it (``Stage.backward_event``), the
    last stage's with an event recorded behind ``loss_fn``, so a backward pass waits for its data and for nothing else.  ``step`` returns the per-micro-batch losses (``losses[-1]`` is the reference's ``_loss_fn``,
    bert/graph.py:166); weight gradients accumulate in each stage's ``grads``; ``all_outputs[j][i]`` keeps the boundary
    tensor of micro-batch j leaving stage i, like the reference's list of the same name."""

    def __init__(self, stages, num_micro_batches, loss_fn, variant="S"):
        self.stages, self.m, self.loss_fn = list(stages), num_micro_batches, loss_fn
        S = len(self.stages)
        self.ops = [schedule_ops(i, S, num_micro_batches, variant) for i in range(S)]
        for i, st in enumerate(self.stages):
            k = min(stash_depth(i, S, variant), num_micro_batches)
            if st.stash_slots < k:
                raise ValueError("stage %d has %d stash slots, the schedule needs %d" % (i, st.stash_slots, k))
            if i > 0 and st.in_numel != self.stages[i - 1].out_numel:
                raise ValueError("stage %d takes %d elements, stage %d hands over %d" % (i, st.in_numel, i - 1, self.stages[i - 1].out_numel))
        self.issued = []          # (stage, op, micro-batch) in issue order, for inspection

    def step(self, inputs, key_masks=None):
        S, M = len(self.stages), self.m
        if len(inputs) != M:
            raise ValueError("expected %d micro-batches" % M)
        dev = inputs[0].device
        self.all_outputs = [[torch.empty(st.out_numel, dtype=st.act_dtype, device=dev) for st in self.stages] for _ in range(M)]
        in_grads = [[torch.empty(st.in_numel, dtype=st.act_dtype, device=dev) if st.takes_input_grad else None
                     for st in self.stages] for _ in range(M)]
        d_last = [None] * M
        d_ready = [None] * M
        bwd_event = [dict() for _ in range(S)]
        losses = [None] * M
        fdone = [[False] * M for _ in range(S)]
        bdone = [[False] * M for _ in range(S)]
        cursor = [0] * S
        slot_of = [dict() for _ in range(S)]
        free = [list(range(st.stash_slots)) for st in self.stages]
        self.issued = []
        remaining = sum(len(o) for o in self.ops)
        while remaining:
            progressed = False
            for i, st in enumerate(self.stages):
                while cursor[i] < len(self.ops[i]):
                    op, j = self.ops[i][cursor[i]]
                    if op == "F":
                        if i > 0 and not fdone[i - 1][j]:
                            break
                        slot = free[i].pop(0)
                        slot_of[i][j] = slot
                        x = inputs[j] if i == 0 else self.all_outputs[j][i - 1]
                        st.forward(slot, x, self.all_outputs[j][i], None if key_masks is None else key_masks[j])
                        fdone[i][j] = True
                        if i == S - 1:
                            losses[j], d_last[j] = self.loss_fn(j, self.all_outputs[j][i])
                            d_ready[j] = torch.cuda.Event()
                            d_ready[j].record()
                    else:
                        if i < S - 1 and not bdone[i + 1][j]:
                            break
                        d_out = d_last[j] if i == S - 1 else in_grads[j][i + 1]
                        slot = slot_of[i].pop(j)
                        if i == S - 1:
                            ready = d_ready[j]
                        else:
                            # the pass of the next stage that wrote d_out: its event if it ran on a stream of its own
                            # (read before that slot is used again), else the order of the shared stream
                            ready = bwd_event[i + 1].pop(j)
                            if ready is None:
                                ready = False
                        st.backward(slot, d_out.reshape(-1), in_grads[j][i], ready=ready)
                        bwd_event[i][j] = st.backward_event(slot)
                        free[i].append(slot)
                        bdone[i][j] = True
                    self.issued.append((i, op, j))
                    cursor[i] += 1
                    remaining -= 1
                    progressed = True
            if not progressed:
                raise RuntimeError("pipeline schedule cannot make progress")
        for st in self.stages:
            st.join()
        return losses
