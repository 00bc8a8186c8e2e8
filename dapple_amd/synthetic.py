"""Seeded synthetic inputs, weights and upstream gradients for the stage configs.

Every array comes from ``numpy.random.Generator(PCG64(seed))``: inputs use seed
1000+config, weights 2000+config, upstream gradients 3000+config, and micro-batch
``m`` adds ``m`` to the seed, so a CPU checker and the GPU stage see identical
bits without exchanging files.

Weight keys follow the reference's TF variable scopes
(bert/models/bert/modeling_slice.py:945-996), so a checkpoint name map applies
unchanged.
"""
import numpy as np

SEED_INPUT = 1000
SEED_WEIGHT = 2000
SEED_GRAD = 3000


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


# --------------------------------------------------------------------------- BERT
def bert_layer_shapes(hidden, ffn):
    """Per-encoder-layer variable shapes, in the reference's scope order."""
    return [
        ("attention/self/query/kernel", (hidden, hidden)),
        ("attention/self/query/bias", (hidden,)),
        ("attention/self/key/kernel", (hidden, hidden)),
        ("attention/self/key/bias", (hidden,)),
        ("attention/self/value/kernel", (hidden, hidden)),
        ("attention/self/value/bias", (hidden,)),
        ("attention/output/dense/kernel", (hidden, hidden)),
        ("attention/output/dense/bias", (hidden,)),
        ("attention/output/LayerNorm/gamma", (hidden,)),
        ("attention/output/LayerNorm/beta", (hidden,)),
        ("intermediate/dense/kernel", (hidden, ffn)),
        ("intermediate/dense/bias", (ffn,)),
        ("output/dense/kernel", (ffn, hidden)),
        ("output/dense/bias", (hidden,)),
        ("output/LayerNorm/gamma", (hidden,)),
        ("output/LayerNorm/beta", (hidden,)),
    ]


def bert_embedding_shapes(vocab, hidden, type_vocab, max_pos):
    return [
        ("bert/embeddings/word_embeddings", (vocab, hidden)),
        ("bert/embeddings/token_type_embeddings", (type_vocab, hidden)),
        ("bert/embeddings/position_embeddings", (max_pos, hidden)),
        ("bert/embeddings/LayerNorm/gamma", (hidden,)),
        ("bert/embeddings/LayerNorm/beta", (hidden,)),
    ]


def bert_weights(seed, num_layers, hidden, ffn, first_layer=0, embeddings=None,
                 stddev=0.02, perturb=False):
    """N(0, stddev) kernels/tables, zero biases, LayerNorm gamma 1 / beta 0.

    ``perturb=True`` draws biases, gamma and beta at random too, so that a test
    can tell a dropped bias or a swapped gamma/beta apart from a correct result.
    ``embeddings`` = (vocab, type_vocab, max_pos) adds the embedding tables.
    """
    rng = _rng(seed)
    w = {}

    def fill(name, shape):
        if name.endswith("kernel") or name.endswith("embeddings"):
            w[name] = (rng.standard_normal(shape) * stddev).astype(np.float32)
        elif name.endswith("gamma"):
            w[name] = (1.0 + 0.1 * rng.standard_normal(shape)).astype(np.float32) if perturb \
                else np.ones(shape, np.float32)
        else:
            w[name] = (0.1 * rng.standard_normal(shape)).astype(np.float32) if perturb \
                else np.zeros(shape, np.float32)

    if embeddings is not None:
        vocab, type_vocab, max_pos = embeddings
        for name, shape in bert_embedding_shapes(vocab, hidden, type_vocab, max_pos):
            fill(name, shape)
    for l in range(first_layer, first_layer + num_layers):
        for name, shape in bert_layer_shapes(hidden, ffn):
            fill("bert/encoder/layer_%d/%s" % (l, name), shape)
    return w


def bert_activation_inputs(seed, num_micro_batches, batch, seq, hidden):
    """Stage-boundary activations N(0,1), one [batch*seq, hidden] per micro-batch."""
    return [_rng(seed + m).standard_normal((batch * seq, hidden)).astype(np.float32)
            for m in range(num_micro_batches)]


def bert_id_inputs(seed, num_micro_batches, batch, seq, vocab):
    return [_rng(seed + m).integers(0, vocab, size=(batch, seq)).astype(np.int32)
            for m in range(num_micro_batches)]


def upstream_grads(seed, num_micro_batches, shape):
    return [_rng(seed + m).standard_normal(shape).astype(np.float32)
            for m in range(num_micro_batches)]


# --------------------------------------------------------------------------- VGG19
# (name, out_channels | None for a 2x2 max-pool) in the order a stage-0 replica applies them
# (vgg19/applications/vgg19_slice_model.py:280-302); the 15:1 split of the reference ends at
# block5_conv2, BASELINE configs[1] runs the whole conv stack.
VGG19_STAGE0_15_1 = [
    ("block1_conv1", 64), ("block1_conv2", 64), ("block1_pool", None),
    ("block2_conv1", 128), ("block2_conv2", 128), ("block2_pool", None),
    ("block3_conv1", 256), ("block3_conv2", 256), ("block3_conv3", 256), ("block3_conv4", 256), ("block3_pool", None),
    ("block4_conv1", 512), ("block4_conv2", 512), ("block4_conv3", 512), ("block4_conv4", 512), ("block4_pool", None),
    ("block5_conv1", 512), ("block5_conv2", 512),
]
VGG19_CONV_STACK = VGG19_STAGE0_15_1 + [("block5_conv3", 512), ("block5_conv4", 512)]
# what the last device runs in front of the classification block (vgg19_slice_model.py:327-340): with 15 replicas only the end
# of block 5, with 2 replicas blocks 4 and 5
VGG19_STAGE1_15_1 = [("block5_conv3", 512), ("block5_conv4", 512), ("block5_pool", None)]
VGG19_STAGE1_2_1 = VGG19_STAGE0_15_1[11:] + VGG19_STAGE1_15_1


def vgg_weights(seed, layers, in_channels=3, perturb=False):
    """He-normal kernels (sigma = sqrt(2 / (9 Cin))), HWIO [3,3,Cin,Cout]; biases 0 (or random)."""
    rng = _rng(seed)
    w, cin = {}, in_channels
    for name, cout in layers:
        if cout is None:
            continue
        w[name + "/kernel"] = (rng.standard_normal((3, 3, cin, cout)) * np.sqrt(2.0 / (9 * cin))).astype(np.float32)
        w[name + "/bias"] = (0.1 * rng.standard_normal(cout)).astype(np.float32) if perturb else np.zeros(cout, np.float32)
        cin = cout
    return w


def vgg_head_weights(seed, features, fc=4096, classes=1000, perturb=False):
    """fc1 / fc2 / predictions of vgg19_slice_model.py:218-220 under keras' Dense defaults: glorot-uniform kernels
    [in, out], zero biases (or small random ones)."""
    rng = _rng(seed)
    w = {}
    for name, (i, o) in (("fc1", (features, fc)), ("fc2", (fc, fc)), ("predictions", (fc, classes))):
        lim = np.sqrt(6.0 / (i + o))
        w[name + "/kernel"] = rng.uniform(-lim, lim, (i, o)).astype(np.float32)
        w[name + "/bias"] = (0.1 * rng.standard_normal(o)).astype(np.float32) if perturb else np.zeros(o, np.float32)
    return w


def vgg_inputs(seed, num_micro_batches, batch, height, width, channels=3):
    return [_rng(seed + m).standard_normal((batch, height, width, channels)).astype(np.float32)
            for m in range(num_micro_batches)]


def vgg_layers(channels):
    """[(keras-style name, out_channels | None)] for a list like [64, 64, None, 128]: convs are named
    block%d_conv%d and pools block%d_pool, the block index growing after every pool."""
    out, block, k = [], 1, 0
    for c in channels:
        if c is None:
            out.append(("block%d_pool" % block, None))
            block, k = block + 1, 0
        else:
            k += 1
            out.append(("block%d_conv%d" % (block, k), c))
    return out


def scale_layers(layers, divisor):
    """Same topology with every channel count divided (reduced-size fixtures and tests)."""
    return [(n, None if c is None else max(c // divisor, 1)) for n, c in layers]


# --------------------------------------------------------------------------- GNMT encoder
GNMT_SCOPE = "dynamic_seq2seq/encoder/"


def gnmt_cell_scopes(num_layers):
    """Variable scopes of the encoder's LSTM cells (gnmt/nmt/gnmt_model.py:96-166): the fw and bw cell
    of the bidirectional layer, then uni layers 1..num_layers-1."""
    s = [GNMT_SCOPE + "bidirectional_rnn/fw/basic_lstm_cell", GNMT_SCOPE + "bidirectional_rnn/bw/basic_lstm_cell"]
    s += [GNMT_SCOPE + "rnn/multi_rnn_cell/cell_%d/rnn/basic_lstm_cell" % l for l in range(1, num_layers)]
    return s


def gnmt_weights(seed, num_layers, units, vocab, init_weight=0.1, perturb=False):
    """U(-init_weight, init_weight) embedding table and LSTM kernels [in+units, 4*units]; biases 0."""
    rng = _rng(seed)
    w = {GNMT_SCOPE + "embedding_encoder": rng.uniform(-init_weight, init_weight, (vocab, units)).astype(np.float32)}
    for i, scope in enumerate(gnmt_cell_scopes(num_layers)):
        n_in = 2 * units if i == 2 else units           # uni layer 1 reads the fw|bw concatenation
        w[scope + "/kernel"] = rng.uniform(-init_weight, init_weight, (n_in + units, 4 * units)).astype(np.float32)
        w[scope + "/bias"] = rng.uniform(-init_weight, init_weight, 4 * units).astype(np.float32) if perturb \
            else np.zeros(4 * units, np.float32)
    return w


def gnmt_id_inputs(seed, num_micro_batches, batch, seq, vocab):
    return [_rng(seed + m).integers(0, vocab, size=(batch, seq)).astype(np.int32) for m in range(num_micro_batches)]


# --------------------------------------------------------------------------- XLNet
def xlnet_layer_shapes(hidden, heads, ffn):
    """Per-layer tensors of an XLNet layer (xlnet/layers/rel_multihead_attn.py:35-67, rel_bias.py:30-63,
    segment_embed.py:23-31, position_wise_feed_forward.py:56-90, layer_normalization.py:47-67); q/k/v/r/o are
    [hidden, heads, head_dim] flattened to [hidden, hidden]; the [num_layer, ...] bias and segment tables
    of the reference are held one slice per layer."""
    return [("q", (hidden, hidden)), ("k", (hidden, hidden)), ("v", (hidden, hidden)), ("r", (hidden, hidden)),
            ("o", (hidden, hidden)), ("bias_context", (hidden,)), ("bias_relative", (hidden,)), ("bias_segment", (hidden,)),
            ("seg_emb", (2, hidden)), ("attn_ln/gamma", (hidden,)), ("attn_ln/beta", (hidden,)),
            ("ff/W1", (hidden, ffn)), ("ff/b1", (ffn,)), ("ff/W2", (ffn, hidden)), ("ff/b2", (hidden,)),
            ("ff_ln/gamma", (hidden,)), ("ff_ln/beta", (hidden,))]


def xlnet_weights(seed, num_layers, hidden, heads, ffn, first_layer=0, stddev=0.02, perturb=False):
    rng = _rng(seed)
    w = {}
    for l in range(first_layer, first_layer + num_layers):
        for name, shape in xlnet_layer_shapes(hidden, heads, ffn):
            key = "layer_%d/%s" % (l, name)
            if name.endswith("gamma"):
                w[key] = (1 + 0.1 * rng.standard_normal(shape)).astype(np.float32) if perturb else np.ones(shape, np.float32)
            elif name.endswith("beta") or name in ("ff/b1", "ff/b2"):
                w[key] = (0.1 * rng.standard_normal(shape)).astype(np.float32) if perturb else np.zeros(shape, np.float32)
            else:
                w[key] = (rng.standard_normal(shape) * stddev).astype(np.float32)
    return w


def xlnet_perm_masks(seed, qlen, mlen, batch):
    """Content- and query-stream masks [qlen, mlen+qlen, batch] (1 = masked) of a random factorization
    order: position i sees j when j comes no later (content) / strictly earlier (query) in the order;
    memory is always visible."""
    rng = _rng(seed)
    mh = np.zeros((qlen, mlen + qlen, batch), np.float32)
    mg = np.zeros_like(mh)
    for b in range(batch):
        rank = np.empty(qlen, np.int64)
        rank[rng.permutation(qlen)] = np.arange(qlen)
        mh[:, mlen:, b] = (rank[None, :] > rank[:, None]).astype(np.float32)
        mg[:, mlen:, b] = (rank[None, :] >= rank[:, None]).astype(np.float32)
    return mh, mg


def xlnet_stream_inputs(seed, num_micro_batches, qlen, batch, hidden, streams=2):
    return [[_rng(seed + m + 100 * s).standard_normal((qlen, batch, hidden)).astype(np.float32) for s in range(streams)]
            for m in range(num_micro_batches)]


def xlnet_mems(seed, num_layers, mlen, batch, hidden):
    return [_rng(seed + 7 * l).standard_normal((mlen, batch, hidden)).astype(np.float32) for l in range(num_layers)]


# --------------------------------------------------------------------------- configs
CONFIGS = {
    # BASELINE configs[0]: BERT-Large 2-layer encoder stage behind the embedding
    "bert_large_2l": dict(index=0, kind="bert", num_layers=2, hidden=1024, heads=16, ffn=4096,
                          seq=128, micro_batch=2, num_micro_batches=4, dtype="fp32",
                          embeddings=(30522, 2, 512)),
    # BASELINE configs[1]: VGG19 conv stack (stage 0 of the 15:1 split, widened to conv5_4)
    "vgg19_stage0": dict(index=1, kind="vgg", layers=VGG19_CONV_STACK, height=224, width=224, in_channels=3,
                         micro_batch=32, num_micro_batches=4, dtype="fp32"),
    # VGG19's last device in the 15:1 split (not a BASELINE configuration: a last-stage row): block5_conv3, block5_conv4,
    # block5_pool on the concatenated boundary activation, then flatten, fc1, fc2, predictions and the loss
    "vgg19_last_device": dict(index=7, kind="vgg_last", layers=VGG19_STAGE1_15_1, height=14, width=14, in_channels=512,
                              fc=4096, classes=1000, micro_batch=32, num_micro_batches=4, dtype="fp32"),
    # BASELINE configs[2]: GNMT-16 encoder stage (8 LSTM layers, the first bidirectional)
    "gnmt16_encoder": dict(index=2, kind="gnmt", num_layers=8, units=1024, vocab=32000, seq=50, micro_batch=64,
                           num_micro_batches=4, dtype="fp32", forget_bias=1.0),
    # GNMT-16's two decoder pieces as the reference places them (not BASELINE configurations: the last-stage rows):
    # decoder cell 0 + attention wrapper behind the encoder on device 0; cells 1..15, projection and loss on device 1
    "gnmt16_attention_cell": dict(index=5, kind="gnmt_attention", units=1024, vocab=32000, seq=50, src_seq=50, micro_batch=64,
                                  num_micro_batches=4, dtype="fp32", forget_bias=1.0),
    "gnmt16_decoder": dict(index=6, kind="gnmt_decoder", num_layers=15, first_layer=1, units=1024, vocab=32000, seq=50,
                           micro_batch=64, num_micro_batches=4, dtype="fp32", forget_bias=1.0),
    # BASELINE configs[3]: BERT-48 half-stage
    "bert48_half": dict(index=3, kind="bert", num_layers=24, hidden=1024, heads=16, ffn=4096,
                        seq=512, micro_batch=2, num_micro_batches=8, dtype="bf16",
                        embeddings=None),
    # BASELINE configs[4]: XLNet-36 half-stage, two streams, memory 384
    "xlnet36_half": dict(index=4, kind="xlnet", num_layers=18, hidden=1024, heads=16, ffn=4096, seq=512, mem_len=384,
                         micro_batch=1, num_micro_batches=8, dtype="bf16", streams=2),
    # one normal cell of the reference driver's AmoebaNet (not a BASELINE configuration): amoeba_net_d, reduction_size 256
    # (amoeba_net/amoeba-dapple.py:132-136), a cell behind the first reduction cell: 28 x 28 maps, 4 x 256 channels in, batch 8
    "amoeba_net_d_cell": dict(index=8, kind="amoeba", cell="amoeba_net_d", filters=256, in_channels=1024, height=28, width=28,
                              micro_batch=8, num_micro_batches=4, dtype="fp32"),
}


def gnmt_decoder_weights(seed, first_layer, num_layers, units, init_weight=0.1, perturb=False):
    """Decoder cells first_layer .. of the second device: kernels [3*units, 4*units] (input | attention | h), biases 0."""
    rng = _rng(seed)
    w = {}
    for l in range(first_layer, first_layer + num_layers):
        scope = "dynamic_seq2seq/decoder/multi_rnn_cell_part2/cell_%d/basic_lstm_cell" % l
        w[scope + "/kernel"] = rng.uniform(-init_weight, init_weight, (3 * units, 4 * units)).astype(np.float32)
        w[scope + "/bias"] = rng.uniform(-init_weight, init_weight, 4 * units).astype(np.float32) if perturb \
            else np.zeros(4 * units, np.float32)
    return w


def gnmt_attention_weights(seed, units, vocab, init_weight=0.1, perturb=False):
    """Decoder cell 0 with its attention wrapper: embedding_decoder, the cell's kernel [3*units, 4*units] and bias, the
    memory and query layers, attention_v, attention_g (sqrt(1/units), TensorFlow's initial value) and attention_b."""
    rng = _rng(seed)
    P = "dynamic_seq2seq/decoder/"
    A = P + "multi_rnn_cell_part1/cell_0_attention/attention/"
    u = lambda *shape: rng.uniform(-init_weight, init_weight, shape).astype(np.float32)
    return {P + "embedding_decoder": u(vocab, units),
            A + "basic_lstm_cell/kernel": u(3 * units, 4 * units),
            A + "basic_lstm_cell/bias": u(4 * units) if perturb else np.zeros(4 * units, np.float32),
            P + "memory_layer/kernel": u(units, units),
            A + "bahdanau_attention/query_layer/kernel": u(units, units),
            A + "bahdanau_attention/attention_v": u(units),
            A + "bahdanau_attention/attention_g": np.array([np.sqrt(1.0 / units) * (1.3 if perturb else 1.0)], np.float32),
            A + "bahdanau_attention/attention_b": u(units) if perturb else np.zeros(units, np.float32)}


# ---- AmoebaNet cells (amoeba_net/model_specs.py:22-87: normal cells of the four published networks)
AMOEBA_NORMAL_CELLS = {
    "amoeba_net_a": (["avg_pool_3x3", "max_pool_3x3", "separable_3x3_2", "none", "none", "avg_pool_3x3", "separable_3x3_2",
                      "separable_5x5_2", "avg_pool_3x3", "separable_3x3_2"], [0, 0, 1, 1, 0, 1, 0, 2, 5, 0], [1, 0, 1, 0, 0, 1, 0]),
    "amoeba_net_b": (["1x1", "max_pool_3x3", "none", "separable_3x3_2", "1x1", "separable_3x3_2", "1x1", "none", "avg_pool_3x3",
                      "1x1"], [1, 1, 1, 0, 1, 0, 2, 2, 1, 5], [0, 1, 1, 0, 0, 1, 0]),
    "amoeba_net_c": (["avg_pool_3x3", "separable_3x3_2", "none", "separable_3x3_2", "avg_pool_3x3", "separable_3x3_2", "none",
                      "separable_3x3_2", "avg_pool_3x3", "separable_3x3_2"], [0, 0, 0, 0, 2, 1, 0, 1, 3, 0], [1, 0, 0, 1, 0, 0, 0]),
    "amoeba_net_d": (["1x1", "max_pool_3x3", "none", "1x7_7x1", "1x1", "1x7_7x1", "max_pool_3x3", "none", "avg_pool_3x3", "1x1"],
                     [1, 1, 1, 0, 0, 0, 2, 2, 1, 5], [0, 1, 1, 0, 0, 1, 0]),
}


def amoeba_cell_weights(seed, shapes, perturb=True):
    """name -> fp32 array for the shapes of ``dapple_amd.amoeba.cell_variable_shapes``: kernels from a variance-scaling normal
    (fan-out), gamma = 1, beta = 0 (perturbed on request so their gradients are exercised), moving statistics at their
    initial 0 / 1."""
    rng = _rng(seed)
    w = {}
    for name in sorted(shapes):
        shp = shapes[name]
        if name.endswith("gamma"):
            w[name] = (1 + 0.2 * rng.standard_normal(shp)).astype(np.float32) if perturb else np.ones(shp, np.float32)
        elif name.endswith("beta"):
            w[name] = (0.2 * rng.standard_normal(shp)).astype(np.float32) if perturb else np.zeros(shp, np.float32)
        elif name.endswith("moving_mean"):
            w[name] = np.zeros(shp, np.float32)
        elif name.endswith("moving_variance"):
            w[name] = np.ones(shp, np.float32)
        else:
            fan_out = shp[-1] if not name.endswith("depthwise_weights") else shp[0] * shp[1]
            w[name] = (rng.standard_normal(shp) * np.sqrt(2.0 / fan_out)).astype(np.float32)
    return w
