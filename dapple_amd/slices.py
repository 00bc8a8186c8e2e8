"""Host-side mirror of the reference's stage-slice interfaces, on top of the HIP stage runtime.

Same class / function names, argument names and error behaviour as the reference's slice files, so
a driver written against them finds what it expects; what they return are GPU tensors computed
eagerly through ``libdapple_hip.so`` instead of TF graph symbols.

    BertConfig, BertModelSlice          bert/models/bert/modeling_slice.py:646-717, 722-1009
    BertFinetuneSlice                   bert/models/bert/bert.py:385-479 (calc_device :419-430)
    SliceVGG19                          vgg19/applications/vgg19_slice_model.py:38-357
    XlnetSlice                          xlnet/models/slice_xlnet.py:22-246 (calc_device :106-121)
    _single_cell_dapple, GNMTEncoderSlice   gnmt/nmt/model_helper.py:399-456, gnmt_model.py:61-221
    calc_reduction_layers, BaseCell, build_network   amoeba_net/network_utils_slice.py:83-90, 294-313,
                                        model_builder_slice.py:292-345 (API shell: no config runs it)

``dep_outputs`` arguments are accepted and ignored on purpose: in the reference they only add TF
control dependencies (values unused, bert.py:439-449); here ordering is the launch order that
``dapple_amd.runtime.StageRuntime`` issues.
"""
import copy
import json
import sys

import torch

from . import runtime, synthetic


# =========================================================================== BERT
class BertConfig(object):
    """Configuration for `BertModel` (modeling_slice.py:646-717)."""

    def __init__(self, vocab_size, hidden_size=768, num_hidden_layers=12, num_attention_heads=12,
                 intermediate_size=3072, hidden_act="gelu", hidden_dropout_prob=0.1,
                 attention_probs_dropout_prob=0.1, max_position_embeddings=512, type_vocab_size=16,
                 initializer_range=0.02):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.num_hidden_layers = num_hidden_layers
        self.num_attention_heads = num_attention_heads
        self.hidden_act = hidden_act
        self.intermediate_size = intermediate_size
        self.hidden_dropout_prob = hidden_dropout_prob
        self.attention_probs_dropout_prob = attention_probs_dropout_prob
        self.max_position_embeddings = max_position_embeddings
        self.type_vocab_size = type_vocab_size
        self.initializer_range = initializer_range

    @classmethod
    def from_dict(cls, json_object):
        config = BertConfig(vocab_size=None)
        for (key, value) in json_object.items():
            config.__dict__[key] = value
        return config

    @classmethod
    def from_json_file(cls, json_file):
        with open(json_file, "r") as reader:
            text = reader.read()
        return cls.from_dict(json.loads(text))

    def to_dict(self):
        return copy.deepcopy(self.__dict__)

    def to_json_string(self):
        return json.dumps(self.to_dict(), indent=2, sort_keys=True) + "\n"


class BertModelSlice(object):
    """``stages`` = [embedding_stage, reshape_input, layer_0 .. layer_{L-1}, pooler_stage]
    (modeling_slice.py:792, 823, 837, 870), each ``f(prev_output, *args) -> tensor``.

    ``weights`` maps the reference's variable names to arrays; absent, N(0, initializer_range) /
    zeros / ones are drawn from ``seed``.  ``dtype`` is the compute type ("fp32" or "bf16")."""

    def __init__(self, config, is_training, input_ids, input_mask=None, token_type_ids=None,
                 use_one_hot_embeddings=True, scope=None, weights=None, dtype="fp32", seed=0):
        config = copy.deepcopy(config)
        if not is_training:
            config.hidden_dropout_prob = 0.0
            config.attention_probs_dropout_prob = 0.0
        if config.hidden_dropout_prob or config.attention_probs_dropout_prob:
            raise ValueError("dropout is not part of this runtime: build the model with is_training=False "
                             "or zero dropout probabilities")
        if config.hidden_act != "gelu":
            raise ValueError("Unsupported activation: %s" % config.hidden_act)
        if input_ids.dim() != 2:
            raise ValueError("For the tensor `input_ids`, the actual rank `%d` (shape = %s) is not equal to the "
                             "expected rank `2`" % (input_ids.dim(), tuple(input_ids.shape)))
        if config.hidden_size % config.num_attention_heads != 0:
            raise ValueError("The hidden size (%d) is not a multiple of the number of attention heads (%d)"
                             % (config.hidden_size, config.num_attention_heads))
        self.config, self.dtype = config, dtype
        self.batch_size, self.seq_length = input_ids.shape
        if self.seq_length > config.max_position_embeddings:
            raise ValueError("The seq length (%d) cannot be greater than `max_position_embeddings` (%d)"
                             % (self.seq_length, config.max_position_embeddings))
        self.input_ids = input_ids.to(torch.int32).contiguous()
        if input_mask is None:
            input_mask = torch.ones_like(self.input_ids)
        if token_type_ids is None:
            token_type_ids = torch.zeros_like(self.input_ids)
        self.input_mask = input_mask
        self.token_type_ids = token_type_ids.to(torch.int32).contiguous()
        # [B, F, T] float mask of modeling_slice.py:323-354; the kernels take its [B, T] key form
        self.attention_mask = torch.ones(self.batch_size, self.seq_length, 1, device=input_ids.device) * \
            input_mask.reshape(self.batch_size, 1, self.seq_length).float()
        self._key_mask = None if bool((input_mask != 0).all()) else input_mask.float().contiguous()
        emb = (config.vocab_size, config.type_vocab_size, config.max_position_embeddings)
        self.weights = weights if weights is not None else synthetic.bert_weights(
            seed, config.num_hidden_layers, config.hidden_size, config.intermediate_size, embeddings=emb,
            stddev=config.initializer_range)
        self.all_encoder_layers = []
        self.sequence_output = self.embedding_output = self.pooled_output = None
        self._handles = {}

        def embedding_stage(*args):
            st = self._op_stage("emb")
            out = torch.empty(self.batch_size * self.seq_length, config.hidden_size, dtype=st.act_dtype, device=input_ids.device)
            st.forward(0, self.input_ids, out, token_type_ids=self.token_type_ids)
            st.release(0)
            self.embedding_output = out.reshape(self.batch_size, self.seq_length, config.hidden_size)
            return self.embedding_output

        def reshape_input(input_tensor, *args):
            if input_tensor.dim() != 3:
                raise ValueError("For the tensor `input_tensor`, the actual rank `%d` is not equal to the expected rank `3`"
                                 % input_tensor.dim())
            self.input_shape = list(input_tensor.shape)
            if self.input_shape[2] != config.hidden_size:
                raise ValueError("The width of the input tensor (%d) != hidden size (%d)" % (self.input_shape[2], config.hidden_size))
            return input_tensor.reshape(-1, config.hidden_size)

        def create_layer(idx):
            def encoder_layer(layer_input, *args):
                st = self._op_stage(idx)
                out = torch.empty_like(layer_input)
                st.forward(0, layer_input.contiguous(), out, key_mask=self._key_mask)
                st.release(0)
                final = out.reshape(self.batch_size, self.seq_length, config.hidden_size)
                self.all_encoder_layers.append(final)
                self.sequence_output = final
                return out
            return encoder_layer

        def pooler_stage(sequence_output, *args):
            # modeling_slice.py:849-868: tanh dense (bert/pooler/dense) on the first token of every sample
            from . import ops
            if self.sequence_output is None:
                self.sequence_output = sequence_output
            x = self.sequence_output.reshape(self.batch_size * self.seq_length, config.hidden_size).contiguous()
            kernel, bias = self._pooler_params(x.device)
            self.pooled_output = ops.pooler(x, self.batch_size, self.seq_length, kernel, bias)
            return self.pooled_output

        self.stages = [embedding_stage, reshape_input]
        self.stages += [create_layer(i) for i in range(config.num_hidden_layers)]
        self.stages.append(pooler_stage)

    def _pooler_params(self, device):
        """bert/pooler/dense/{kernel, bias} from ``weights`` when present, else truncated-normal-like N(0, initializer_range)
        and zeros (modeling_slice.py:862-866) drawn once."""
        if getattr(self, "_pooler", None) is None:
            H = self.config.hidden_size
            if "bert/pooler/dense/kernel" in self.weights:
                k = torch.as_tensor(self.weights["bert/pooler/dense/kernel"], dtype=torch.float32)
                b = torch.as_tensor(self.weights["bert/pooler/dense/bias"], dtype=torch.float32)
            else:
                g = torch.Generator().manual_seed(4321)
                k = torch.randn(H, H, generator=g) * self.config.initializer_range
                b = torch.zeros(H)
            self._pooler = (k.to(device).contiguous(), b.to(device).contiguous())
        return self._pooler

    def _op_stage(self, which):
        """A one-op stage handle (the embedding, or encoder layer ``which``), created on first use."""
        if which not in self._handles:
            c = self.config
            if which == "emb":
                st = runtime.bert_stage(0, c.hidden_size, c.num_attention_heads, c.intermediate_size, self.batch_size,
                                        self.seq_length, self.dtype, 1,
                                        embeddings=(c.vocab_size, c.type_vocab_size, c.max_position_embeddings))
            else:
                st = runtime.bert_stage(1, c.hidden_size, c.num_attention_heads, c.intermediate_size, self.batch_size,
                                        self.seq_length, self.dtype, 1, first_layer=which)
            st.bind(self.weights)
            self._handles[which] = st
        return self._handles[which]

    def get_pooled_output(self):
        return self.pooled_output

    def get_sequence_output(self):
        return self.sequence_output

    def get_all_encoder_layers(self):
        return self.all_encoder_layers

    def get_embedding_output(self):
        return self.embedding_output

    def get_embedding_table(self):
        return self.weights["bert/embeddings/word_embeddings"]


def bert_calc_device(i, nstage):
    """Stage -> device map of bert.py:419-430: BERT-24 (27 stages) splits 11:13 encoder layers, BERT-48 (51
    stages) 23:25; anything else ends the process like the reference (sys.exit(0))."""
    if nstage == 27:
        return 0 if i < 13 else 1
    elif nstage == 51:
        return 0 if i < 25 else 1
    print("Unrecognized nstage, only bert-24 and bert-48 are supported.")
    sys.exit(0)


class BertFinetuneSlice(object):
    """Places ``model.stages`` on the pipeline devices and builds the HIP stage of ``local_device``
    (bert.py:390-456).  ``stage`` is a ``runtime.Stage`` holding every op the planner put on that device."""

    def __init__(self, bert_config_file, max_seq_length, is_training, input_ids, input_mask, segment_ids, labels,
                 use_one_hot_embeddings, model_type='classification', slice_devices="/device:GPU:0",
                 dep_outputs=None, kwargs=None, local_device=0, dtype="bf16", stash_slots=None, weights=None, seed=0):
        bert_config = bert_config_file if isinstance(bert_config_file, BertConfig) else BertConfig.from_json_file(bert_config_file)
        if max_seq_length > bert_config.max_position_embeddings:
            raise ValueError("Cannot use sequence length %d because the BERT model was only trained up to sequence "
                             "length %d" % (max_seq_length, bert_config.max_position_embeddings))
        self.devices = slice_devices if isinstance(slice_devices, list) else slice_devices.split(",")
        self.bert_config, self.kwargs, self.labels, self.input_ids = bert_config, kwargs, labels, input_ids
        L = bert_config.num_hidden_layers
        nstage = L + 3
        self.device_of = [bert_calc_device(i, nstage) for i in range(nstage)]
        mine = [i for i in range(nstage) if self.device_of[i] == local_device]
        layers = [i - 2 for i in mine if 2 <= i < 2 + L]
        with_emb = 0 in mine
        B, S = input_ids.shape
        ndev = max(self.device_of) + 1
        K = stash_slots if stash_slots is not None else runtime.stash_depth(local_device, ndev)
        emb = (bert_config.vocab_size, bert_config.type_vocab_size, bert_config.max_position_embeddings) if with_emb else None
        self.stage = runtime.bert_stage(len(layers), bert_config.hidden_size, bert_config.num_attention_heads,
                                        bert_config.intermediate_size, B, S, dtype, K, embeddings=emb,
                                        first_layer=layers[0] if layers else 0)
        if weights is None:
            weights = synthetic.bert_weights(seed, L, bert_config.hidden_size, bert_config.intermediate_size,
                                             embeddings=(bert_config.vocab_size, bert_config.type_vocab_size,
                                                         bert_config.max_position_embeddings),
                                             stddev=bert_config.initializer_range)
        self.stage.bind(weights)
        self._model_args = (bert_config, is_training, input_ids, input_mask, segment_ids, use_one_hot_embeddings, weights, dtype)
        self._model = None
        self.layers, self.local_device, self.model_type = layers, local_device, model_type
        self.stage_outputs = []
        self.is_last = (nstage - 1) in mine
        self.loss = None
        if self.is_last and model_type == 'mrc':             # bert.py:467-470
            # cls/squad/output_weights [2, hidden] (truncated normal 0.02), output_bias [2] zeros (bert.py:677-683)
            g = torch.Generator().manual_seed(seed + 1)
            H = bert_config.hidden_size
            self.output_weights = (torch.randn(2, H, generator=g) * 0.02).cuda()
            self.output_bias = torch.zeros(2, device="cuda")
            self.d_output_weights = torch.zeros_like(self.output_weights)
            self.d_output_bias = torch.zeros_like(self.output_bias)
        elif self.is_last and model_type in ('classification', 'regression'):   # bert.py:463-466
            # bert/pooler/dense (modeling_slice.py:862-866, truncated normal) and src-output-layer/FC
            # (bert.py:644-652: xavier weights [hidden, 2], biases 1e-4)
            g = torch.Generator().manual_seed(seed + 2)
            H = bert_config.hidden_size
            self.pooler_kernel = (torch.randn(H, H, generator=g) * bert_config.initializer_range).cuda()
            self.pooler_bias = torch.zeros(H, device="cuda")
            nout = 2 if model_type == 'classification' else 1        # num_outputs, bert.py:646 / :619
            limit = (6.0 / (H + nout)) ** 0.5
            self.fc_weights = ((torch.rand(H, nout, generator=g) * 2 - 1) * limit).cuda()
            self.fc_biases = torch.full((nout,), 1e-4, device="cuda")
            self.head_grads = [torch.zeros_like(t) for t in (self.pooler_kernel, self.pooler_bias, self.fc_weights, self.fc_biases)]

    @property
    def model(self):
        """The ``BertModelSlice`` whose ``stages`` this class places on the devices (bert.py:399-408); built on first
        use, over the same weights as ``stage`` (its one-op handles are created as they are called)."""
        if self._model is None:
            cfg, is_training, ids, mask, seg, one_hot, weights, dtype = self._model_args
            self._model = BertModelSlice(config=cfg, is_training=False, input_ids=ids, input_mask=mask, token_type_ids=seg,
                                         use_one_hot_embeddings=one_hot, weights=weights, dtype=dtype)
        return self._model

    @property
    def stages(self):
        """``self.model.stages`` (bert.py:414): the per-op callables [embedding_stage, reshape_input, layer_0 ..,
        pooler_stage]; ``device_of[i]`` is the device ``calc_device`` gives entry i."""
        return self.model.stages

    def build_output_layer_squad(self, sequence_output, is_training=False):
        """bert.py:669-718 on the last device: start / end logits and the SQuAD loss from
        ``kwargs["start_positions"]`` / ``kwargs["end_positions"]``.  Returns the gradient of the loss w.r.t.
        ``sequence_output`` - the upstream gradient of this stage's backward pass; the head's own weight
        gradients are added into ``d_output_weights`` / ``d_output_bias``."""
        from . import ops
        if not (self.is_last and self.model_type == 'mrc'):
            raise ValueError("build_output_layer_squad: this device does not hold the SQuAD output layer")
        B, S = self.input_ids.shape
        sp = torch.as_tensor(self.kwargs["start_positions"], dtype=torch.int32).cuda()
        ep = torch.as_tensor(self.kwargs["end_positions"], dtype=torch.int32).cuda()
        x = sequence_output.reshape(B * S, self.bert_config.hidden_size)
        self.loss, self.start_logits, self.end_logits, dx = ops.squad_head(
            x, B, S, self.output_weights, self.output_bias, sp, ep, self.d_output_weights, self.d_output_bias)
        self.stage_outputs = [sequence_output, self.loss]
        return dx


    def build_output_layer_classification(self, sequence_output):
        """pooler_stage (modeling_slice.py:849-868) and bert.py:642-664 on the last device: pooled output, logits over
        the two classes, loss = mean sparse softmax cross entropy of ``labels`` + the FC weights' l2 regulariser (1e-3).
        Returns the gradient of the loss w.r.t. ``sequence_output`` (non-zero on each sample's first token only); the
        head's weight gradients are added into ``head_grads``."""
        from . import ops
        if not (self.is_last and self.model_type == 'classification'):
            raise ValueError("build_output_layer_classification: this device does not hold the classification layer")
        B, S = self.input_ids.shape
        y = torch.as_tensor(self.labels, dtype=torch.int32).cuda()
        x = sequence_output.reshape(B * S, self.bert_config.hidden_size)
        self.loss, self.logits, self.pooled_output, dx = ops.classifier_head(
            x, B, S, self.pooler_kernel, self.pooler_bias, self.fc_weights, self.fc_biases, y, self.head_grads)
        self.predictions = torch.softmax(self.logits, -1)[:, 1]          # bert.py:654
        self.stage_outputs = [sequence_output, self.loss]
        return dx

    def build_output_layer_regression(self, sequence_output):
        """pooler_stage and bert.py:615-640 on the last device: one output per sample, loss = the reference graph's
        ``reduce_mean(pow(prediction - labels, 2))`` (prediction [batch, 1] against the [batch] labels: the mean over every
        pair) + the FC weights' l2 regulariser.  Returns the gradient of the loss w.r.t. ``sequence_output``; the head's
        weight gradients are added into ``head_grads``."""
        from . import ops
        if not (self.is_last and self.model_type == 'regression'):
            raise ValueError("build_output_layer_regression: this device does not hold the regression layer")
        B, S = self.input_ids.shape
        y = torch.as_tensor(self.labels, dtype=torch.float32).cuda()
        x = sequence_output.reshape(B * S, self.bert_config.hidden_size)
        self.loss, self.logits, self.pooled_output, dx = ops.regression_head(
            x, B, S, self.pooler_kernel, self.pooler_bias, self.fc_weights, self.fc_biases, y, self.head_grads)
        self.predictions = self.logits                                     # bert.py:634-635
        self.stage_outputs = [sequence_output, self.loss]
        return dx


# =========================================================================== VGG19
class SliceVGG19(object):
    """vgg19_slice_model.py:38-357.  With ``local_device=0`` ``build`` runs stage 0 (the replicated conv stack) on one
    replica's share of the batch and returns ``(None, [stage0_output])`` - the loss is the last device's.  With
    ``local_device=1`` it is the last device (:315-357): the rest of the conv stack, flatten, fc1, fc2, predictions and the
    loss; ``build(stage0_output, label)`` returns ``(loss, [stage0_output, loss])`` as the reference does and keeps what
    ``backward`` needs.  ``loss_mode``: "as_written" evaluates the reference's ``K.categorical_crossentropy(x, label)``
    literally (a constant, ``ops.vgg_head``), "sparse_ce" the cross entropy of the label as a class index."""

    def __init__(self, include_top=True, weights='imagenet', input_tensor=None, input_shape=None, pooling=None,
                 classes=1000, num_replica=15, batch_size=None, weight_values=None, seed=0, stash_slots=3, local_device=0,
                 loss_mode="as_written", fc_units=4096, **kwargs):
        if num_replica not in (2, 15):
            print("For VGG19 only 2:1 and 15:1 pipeline are supported currently!")
            sys.exit(-1)
        if local_device not in (0, 1):
            raise ValueError("SliceVGG19: local_device %r (the model has two devices)" % (local_device,))
        if local_device == 1 and not include_top:
            raise ValueError("SliceVGG19: the last device is built with the classification block (include_top=True)")
        self.include_top, self.weights, self.pooling, self.classes = include_top, weights, pooling, classes
        self.num_replica, self.local_device, self.loss_mode, self.fc_units = num_replica, local_device, loss_mode, fc_units
        # 15:1 keeps conv1_1..conv5_2 on stage 0, 2:1 only blocks 1-3 (:280-302); the last device has the rest (:327-340)
        if local_device == 0:
            self.layers = synthetic.VGG19_STAGE0_15_1 if num_replica == 15 else synthetic.VGG19_STAGE0_15_1[:11]
        else:
            self.layers = synthetic.VGG19_STAGE1_15_1 if num_replica == 15 else synthetic.VGG19_STAGE1_2_1
        self._weight_values, self._seed, self._stash = weight_values, seed, stash_slots
        self.stage = None
        self.head_weights = self.head_grads = None

    def _make(self, features):
        n, h, w, c = features.shape
        last = self.local_device == 1
        self.stage = runtime.vgg_stage(self.layers, n, h, w, c, 1 if last else self._stash, need_input_grad=last)
        wv = self._weight_values or synthetic.vgg_weights(self._seed, self.layers, c)
        self.stage.bind({k: v for k, v in wv.items() if not k.startswith(("fc1/", "fc2/", "predictions/"))})
        if last:
            feat = 1
            for d in self.stage.out_shape[1:]:
                feat *= d
            hv = {k: v for k, v in wv.items() if k.startswith(("fc1/", "fc2/", "predictions/"))}
            if not hv:
                hv = synthetic.vgg_head_weights(self._seed + 1, feat, self.fc_units, self.classes)
            self.head_weights = {k: torch.as_tensor(v, dtype=torch.float32).cuda().contiguous() for k, v in hv.items()}
            self.head_grads = {k: torch.zeros_like(v) for k, v in self.head_weights.items()}

    def build(self, features, label, input_shape=None, dep_outputs=None):
        if self.stage is None:
            self._make(features)
        out = torch.empty(self.stage.out_shape, device=features.device)
        self.stage.forward(0, features.contiguous(), out)
        if self.local_device == 0:
            self.stage.release(0)
            return None, [out]
        from . import ops
        labels = torch.as_tensor(label, dtype=torch.float32).reshape(-1).cuda().contiguous()
        self.loss, self.predictions, self._dx = ops.vgg_head(out.reshape(out.shape[0], -1), self.head_weights, labels,
                                                             grads=self.head_grads, loss_mode=self.loss_mode)
        return self.loss, [features, self.loss]

    def backward(self, d_in=None):
        """Last device only: the conv layers' backward pass behind the loss of the latest ``build`` (weight gradients into
        ``stage.grads``; the head's went into ``head_grads`` during ``build``); ``d_in`` receives the gradient of the
        boundary activation for the device before."""
        if self.local_device != 1 or self._dx is None:
            raise ValueError("SliceVGG19.backward: needs the last device and a build() before it")
        self.stage.backward(0, self._dx.reshape(self.stage.out_shape), d_in)
        self._dx = None


# =========================================================================== XLNet
def xlnet_calc_device(i, num_layer):
    """slice_xlnet.py:106-121: stage-function index i (layer l is i = l + 2) -> device; the split is 13
    (XLNet-24: 11 + 13 layers) or 19 (XLNet-36: 17 + 19 layers)."""
    split_layer_id = 13 if num_layer == 24 else 19
    return 0 if i < split_layer_id else 1


class XlnetSlice(object):
    """slice_xlnet.py:22-246: builds the HIP stage holding this device's layers."""

    def __init__(self, num_token, num_layer, num_head, embedding_dim, attention_head_dim, feed_forward_dim, target_len,
                 is_training, memory_len=None, dropout=0.0, attention_dropout=0.0, attention_type=None,
                 shared_biases=True, local_device=0, batch_size=1, dtype="bf16", streams=1, stash_slots=None,
                 weights=None, seed=0):
        if dropout or attention_dropout:
            raise ValueError("dropout is not part of this runtime")
        if num_head * attention_head_dim != embedding_dim:
            raise ValueError("embedding_dim (%d) must equal num_head * attention_head_dim (%d)" % (embedding_dim, num_head * attention_head_dim))
        self.num_layer = num_layer
        layers = [l for l in range(num_layer) if xlnet_calc_device(l + 2, num_layer) == local_device]
        K = stash_slots if stash_slots is not None else runtime.stash_depth(local_device, 2)
        self.layers = layers
        self.stage = runtime.xlnet_stage(len(layers), embedding_dim, num_head, feed_forward_dim, batch_size, target_len, dtype,
                                         K, mem_len=memory_len or 0, streams=streams, first_layer=layers[0])
        w = weights or synthetic.xlnet_weights(seed, len(layers), embedding_dim, num_head, feed_forward_dim, first_layer=layers[0])
        self.stage.bind(w)
        self.is_last = local_device == xlnet_calc_device(num_layer + 2, num_layer)
        if self.is_last:
            # XLnetLoss (losses/xlnet_loss.py:9-34): Dense kernels drawn by keras 'normal' (stddev 0.05), biases 0, LN 1 / 0
            from . import ops
            g = torch.Generator().manual_seed(seed + 7)
            H = embedding_dim
            self.loss_weights = {}
            for name, shape in ((n, f(H)) for n, f in ops.XLNET_HEAD_SHAPES.items()):
                if name in ("start_b", "end_b0", "end_b1", "ans_b0", "ln_beta"):
                    t = torch.zeros(shape)
                elif name == "ln_gamma":
                    t = torch.ones(shape)
                else:
                    t = torch.randn(shape, generator=g) * 0.05
                self.loss_weights[name] = t.cuda()
            self.loss_grads = {n: torch.zeros_like(t) for n, t in self.loss_weights.items()}

    def xlnet_loss(self, cls_index, start_positions, end_positions, is_impossible, p_mask, output, dropout_mask=None):
        """slice_xlnet.py:236-244 on the last device: XLnetLoss on the content stream ``output [seq, batch, hidden]``.
        Sets ``loss`` / ``start_logits`` / ``end_logits`` / ``cls_logits`` and returns the gradient of the loss w.r.t.
        ``output`` - the upstream gradient of this stage's backward pass; the head's weight gradients are added into
        ``loss_grads``.  ``dropout_mask [batch, hidden]``: the factor of the dropout inside the loss (None = ones)."""
        from . import ops
        if not self.is_last:
            raise ValueError("xlnet_loss: this device does not hold the loss layer")
        i32 = lambda t: torch.as_tensor(t, dtype=torch.int32).cuda()
        f32 = lambda t: None if t is None else torch.as_tensor(t, dtype=torch.float32).cuda().contiguous()
        self.loss, self.start_logits, self.end_logits, self.cls_logits, dx = ops.xlnet_squad_head(
            output, self.loss_weights, i32(cls_index), i32(start_positions), i32(end_positions), f32(is_impossible), f32(p_mask),
            f32(dropout_mask), grads=self.loss_grads)
        return dx

    def build(self, inputs, dep_outputs=None, is_training=True):
        """inputs: the boundary activation(s) [streams, seq, batch, hidden]; returns (None, [stage_output])."""
        out = torch.empty(self.stage.out_shape, dtype=self.stage.act_dtype, device=inputs.device)
        self.stage.forward(0, inputs.contiguous(), out)
        self.stage.release(0)
        return None, [out]


# =========================================================================== GNMT
class LSTMCellSpec(object):
    """What ``_single_cell`` describes: BasicLSTMCell(num_units, forget_bias) (+ ResidualWrapper)."""

    def __init__(self, layer_id, num_units, forget_bias, residual_connection, device_str):
        self.layer_id, self.num_units, self.forget_bias = layer_id, num_units, forget_bias
        self.residual_connection, self.device_str = residual_connection, device_str


def _single_cell_dapple(hparams, mode, layer_id, residual_connection=False, device_str=None, residual_fn=None):
    """model_helper.py:399-456.  hparams needs unit_type, num_units, forget_bias, dropout."""
    if hparams.unit_type != "lstm":
        raise ValueError("Unknown unit type %s!" % hparams.unit_type)
    if getattr(hparams, "dropout", 0.0) and mode == "train":
        raise ValueError("dropout is not part of this runtime")
    if residual_fn is not None:
        raise ValueError("custom residual_fn is not supported: the wrapper adds inputs and outputs")
    return LSTMCellSpec(layer_id, hparams.num_units, hparams.forget_bias, residual_connection, device_str)


class GNMTEncoderSlice(object):
    """The encoder stage GNMTModel._build_encoder (gnmt_model.py:61-221) builds under ``dapple_test``:
    cells 0 (fw/bw, no residual), 1 (no residual), 2.. (residual), from ``_single_cell_dapple`` specs."""

    def __init__(self, hparams, batch_size, src_max_len, stash_slots=2, weights=None, seed=0):
        n = hparams.num_encoder_layers
        self.cells = [_single_cell_dapple(hparams, "infer", 0), _single_cell_dapple(hparams, "infer", 0)]
        self.cells += [_single_cell_dapple(hparams, "infer", l, residual_connection=(l >= 2)) for l in range(1, n)]
        self.stage = runtime.gnmt_stage(n, hparams.num_units, hparams.src_vocab_size, batch_size, src_max_len, stash_slots,
                                        forget_bias=hparams.forget_bias)
        self.stage.bind(weights or synthetic.gnmt_weights(seed, n, hparams.num_units, hparams.src_vocab_size,
                                                          init_weight=getattr(hparams, "init_weight", 0.1)))

    def build_graph(self, source_ids, scope=None, dep_outputs=None, source_sequence_length=None):
        out = torch.empty(self.stage.out_shape, device=source_ids.device)
        self.stage.set_lengths(0, None if source_sequence_length is None else
                               source_sequence_length.to(torch.int32).contiguous())
        self.stage.forward(0, source_ids.to(torch.int32).contiguous(), out)
        self.stage.release(0)
        return out


# =========================================================================== AmoebaNet (API shell)
def calc_reduction_layers(num_cells, num_reduction_layers):
    """network_utils_slice.py:83-90."""
    reduction_layers = []
    for pool_num in range(1, num_reduction_layers + 1):
        layer_num = (float(pool_num) / (num_reduction_layers + 1)) * num_cells
        reduction_layers.append(int(layer_num))
    return reduction_layers


class BaseCell(object):
    """network_utils_slice.py:294-428: a NAS cell, cut by the pipeline inside ``cell_3`` (6 cells) / ``cell_7`` (12 cells) with
    two boundary tensors (``cut_outputs``, :335, :365).  Normal cells (stride 1) run on the GPU through ``dapple_amd.amoeba``:
    separable, 1 x k / k x 1 and 1 x 1 convolutions, 3 x 3 average / max pooling, train-mode batch normalisation, the sums of
    the five combinations and the concatenation of the unused states.  TensorFlow keeps a cell's variables in its variable
    scope; here they are handed over with ``bind`` (names as in ``amoeba.cell_variable_shapes``).  Not built: reduction
    cells (stride 2, ``factorized_reduction``), dilated convolutions, drop path with a keep probability below 1 (the
    driver's default is 1.0, amoeba-dapple.py:128)."""

    def __init__(self, num_conv_filters, operations, used_hiddenstates, hiddenstate_indices, drop_path_keep_prob,
                 total_num_cells, drop_path_burn_in_steps, dep_outputs=None):
        self._num_conv_filters, self._operations = num_conv_filters, operations
        self._used_hiddenstates, self._hiddenstate_indices = used_hiddenstates, hiddenstate_indices
        self._drop_path_keep_prob, self._total_num_cells = drop_path_keep_prob, total_num_cells
        self._drop_path_burn_in_steps, self._dep_outputs = drop_path_burn_in_steps, dep_outputs
        self.cut_outputs = []
        # total_num_cells counts the two reduction cells (:580-581); FLAGS.num_cells 6 / 12 put the cut in cell_3 / cell_7 (:309-312)
        self.cut_cell_name = {6: "cell_3", 12: "cell_7"}.get(total_num_cells - 2, "")
        self._variables, self._gradients, self._cells = None, None, []

    def bind(self, variables, gradients=None):
        """``variables`` / ``gradients``: name -> fp32 tensor on the GPU; gradients are added to in place by ``backward``."""
        self._variables, self._gradients = variables, gradients
        return self

    def __call__(self, net, scope=None, filter_scaling=1, stride=1, prev_layer=None, cell_num=-1):
        from . import amoeba
        if self._variables is None:
            raise RuntimeError("BaseCell: bind(variables) before the first call")
        if stride != 1:
            raise NotImplementedError("reduction cells (stride %d) are not built" % stride)
        if self._drop_path_keep_prob < 1.0:
            raise NotImplementedError("drop path with a keep probability below 1 draws from TensorFlow's generator and is not built")
        self._cell_num, self._filter_scaling = cell_num, filter_scaling
        self._filter_size = int(self._num_conv_filters * filter_scaling)
        cell = amoeba.Cell(scope, self._filter_size, self._operations, self._hiddenstate_indices, self._used_hiddenstates,
                           self._variables, self._gradients)
        out = cell.forward(net, prev_layer)
        if scope == self.cut_cell_name:
            self.cut_outputs.extend(cell.cut_outputs)
        self._cells.append(cell)
        return out

    def backward(self, d_out):
        """Backward pass of the latest call not yet walked back: -> (d_net, d_prev_layer or None)."""
        if not self._cells:
            raise RuntimeError("BaseCell.backward without a forward call")
        return self._cells.pop().backward(d_out)


def build_network(inputs, num_classes, is_training=True, hparams=None, dep_outputs=None):
    """model_builder_slice.py:292-345 (signature only): the stem, the reduction cells and the classifier around the cells are
    not built - ``BaseCell`` runs single normal cells."""
    raise NotImplementedError("the AmoebaNet network around the cells (stem, reduction cells, classifier) is not built: "
                              "BaseCell runs single normal cells; none of the measured configurations runs the network")
