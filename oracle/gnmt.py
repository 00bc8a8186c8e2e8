"""CPU restatement of the reference's GNMT encoder stage. TEST INFRASTRUCTURE ONLY.

Follows gnmt/nmt/gnmt_model.py:61-221 (DAPPLE branch: embedding lookup, one bidirectional
layer, uni layer 1 without residual, uni layers 2.. with residual) and
gnmt/nmt/model_helper.py:399-456 (_single_cell: BasicLSTMCell(num_units, forget_bias) +
ResidualWrapper).  BasicLSTMCell itself lives in TensorFlow (un-vendored); its published
algorithm is restated here: one kernel [in+U, 4U] applied to concat([x, h], 1), bias [4U],
gate order i, j, f, o, c' = c*sigmoid(f + forget_bias) + sigmoid(i)*tanh(j),
h' = tanh(c')*sigmoid(o).  tf.nn.dynamic_rnn with full-length sequences is a plain scan from a
zero state; the backward cell of bidirectional_dynamic_rnn scans the reversed sequence.  With
sequence_length (every layer gets iterator.source_sequence_length, gnmt_model.py:103, 223-227)
dynamic_rnn emits zeros and copies the state through for t >= length[b] - the output of the WRAPPED
cell is replaced, so a residual layer emits zeros there too - and the backward direction reverses each
sequence within its own length (tf.reverse_sequence), i.e. it starts from the zero state at
t = length[b] - 1.

Pins (tests/test_oracle_gnmt.py): the cell vs torch.nn.LSTMCell after permuting the gate
blocks (torch order i, f, g, o) and folding forget_bias into the bias; the kernel layout
[in+U, 4U] vs the shape held by gnmt/nmt/model_test.py:86 ((10, 20) for in = U = 5); the
scan vs an explicit Python loop; the bidirectional layer vs torch.nn.LSTM(bidirectional=True); ragged sequences vs torch.nn.LSTM on a
packed sequence (pack_padded_sequence / pad_packed_sequence), both directions.

decoder_part2_forward / nmt_loss restate the second device's share of the decoder (gnmt_model.py:489-537,
model.py:641-686) and the loss (model.py:791-838).  Pins: a two-cell stack vs torch.nn.LSTMCell fed the concatenated
input, with the residual taken from the first half of the input; no gradient reaches the attention input; the loss vs
torch.nn.functional.cross_entropy(reduction="sum") over the unpadded positions divided by the batch size.

attention_cell_forward restates decoder cell 0 under tf.contrib.seq2seq.AttentionWrapper with normed
BahdanauAttention (both un-vendored TensorFlow: "parity unpinned" against TensorFlow itself).  Pins: the LSTM part vs
torch.nn.LSTMCell on concat([x_t, previous attention]); the score by scalar loops on a tiny case; alignments sum to one
over the valid source steps and are exactly zero past them; the context equals torch.bmm(alignments, memory); memory
rows past the source length influence nothing.
"""
import torch

P = "dynamic_seq2seq/encoder/"
EMB = P + "embedding_encoder"


def cell_names(num_layers):
    """[(scope, input_is_concat, residual)] of the LSTM cells of an encoder with num_layers layers."""
    cells = [(P + "bidirectional_rnn/fw/basic_lstm_cell", False, False), (P + "bidirectional_rnn/bw/basic_lstm_cell", False, False)]
    for l in range(1, num_layers):
        cells.append((P + "rnn/multi_rnn_cell/cell_%d/rnn/basic_lstm_cell" % l, l == 1, l >= 2))
    return cells


def lstm_cell(x, h, c, kernel, bias, forget_bias=1.0):
    gates = torch.cat([x, h], 1) @ kernel + bias
    i, j, f, o = gates.chunk(4, 1)
    new_c = c * torch.sigmoid(f + forget_bias) + torch.sigmoid(i) * torch.tanh(j)
    new_h = torch.tanh(new_c) * torch.sigmoid(o)
    return new_h, new_c


def dynamic_rnn(x, kernel, bias, forget_bias=1.0, reverse=False, lengths=None, residual=False):
    """x [T,B,I] time-major, zero initial state -> outputs [T,B,U] (+ x where the cell has a residual wrapper).
    lengths [B] int or None (all full length): steps t >= lengths[b] emit zeros and keep the state."""
    T, B, _ = x.shape
    U = kernel.shape[1] // 4
    h = torch.zeros(B, U, dtype=x.dtype)
    c = torch.zeros(B, U, dtype=x.dtype)
    outs = [None] * T
    order = range(T - 1, -1, -1) if reverse else range(T)
    for t in order:
        nh, nc = lstm_cell(x[t], h, c, kernel, bias, forget_bias)
        out = nh + x[t] if residual else nh             # ResidualWrapper, model_helper.py:445-448
        if lengths is not None:
            live = (t < lengths).to(x.dtype).unsqueeze(1)
            out = out * live
            nh = nh * live + h * (1 - live)
            nc = nc * live + c * (1 - live)
        h, c = nh, nc
        outs[t] = out
    return torch.stack(outs)


def encoder_forward(ids, w, num_layers, forget_bias=1.0, lengths=None):
    """ids [B,T] int -> encoder outputs [T,B,U] (gnmt_model.py:78-210); lengths [B] = source_sequence_length."""
    emb = w[EMB][ids.long().t()]                      # time-major lookup (:78-79, :90-91)
    cells = cell_names(num_layers)
    fw = dynamic_rnn(emb, w[cells[0][0] + "/kernel"], w[cells[0][0] + "/bias"], forget_bias, lengths=lengths)
    bw = dynamic_rnn(emb, w[cells[1][0] + "/kernel"], w[cells[1][0] + "/bias"], forget_bias, reverse=True, lengths=lengths)
    x = torch.cat([fw, bw], -1)                       # :108
    for scope, _, residual in cells[2:]:
        x = dynamic_rnn(x, w[scope + "/kernel"], w[scope + "/bias"], forget_bias, lengths=lengths, residual=residual)
    return x


def to_torch(weights, dtype=torch.float64, requires_grad=False):
    return {k: torch.as_tensor(v).to(dtype).clone().requires_grad_(requires_grad) for k, v in weights.items()}


def stage_vjp(ids, w, d_out, num_layers, forget_bias=1.0, lengths=None):
    names = sorted(w)
    out = encoder_forward(ids, w, num_layers, forget_bias, lengths)
    grads = torch.autograd.grad(out, [w[n] for n in names], grad_outputs=d_out, allow_unused=True)
    return out.detach(), None, {n: g for n, g in zip(names, grads) if g is not None}


# ---- the decoder layers of the second pipeline device and the loss ----
# gnmt_model.py:342-383 (DAPPLE branch): decoder cell 0 with the attention wrapper stays on the encoder device
# (GNMTAttentionMultiCell_1), cells 1.. go to the second device as GNMTAttentionMultiCell_2 (:489-537); cell l has a
# residual wrapper with gnmt_residual_fn for l >= 2 (:346-364).  model.py:641-656 drives part 2 with
# dynamic_decode(BasicDecoder(cell2, TrainingHelper(outputs_1, target_sequence_length), zero state)): without
# impute_finished every step up to the longest target is a plain cell call on the padded input, so it is a scan.
# Each cell reads concat([cur_inp, new_attention]) (:526); new_attention is global_attention[0], a non-trainable
# tf.Variable (:456-459): a constant of the graph - no gradient flows into it - that holds whatever was last assigned
# (its initial value is zero; the assign at :478-479 is fetched by nothing).  Here it is an input, one vector per step.
DP = "dynamic_seq2seq/decoder/multi_rnn_cell_part2/"
PROJ = "build_network/decoder/output_projection/output_projection/kernel"


def decoder_cell_names(first_layer, num_layers):
    """[(scope, residual)] of decoder cells first_layer .. first_layer + num_layers - 1 (variable scope "cell_%d", :521)."""
    return [(DP + "cell_%d/basic_lstm_cell" % l, l >= 2) for l in range(first_layer, first_layer + num_layers)]


def decoder_part2_forward(x, attention, w, first_layer, num_layers, forget_bias=1.0):
    """x [T,B,U]: the outputs of decoder cell 0; attention [T,B,U] or None (zeros) -> outputs of the last cell [T,B,U]."""
    T, B, U = x.shape
    cells = decoder_cell_names(first_layer, num_layers)
    hs = [torch.zeros(B, U, dtype=x.dtype) for _ in cells]         # cell2.zero_state, gnmt_model.py:375
    cs = [torch.zeros(B, U, dtype=x.dtype) for _ in cells]
    outs = []
    for t in range(T):
        cur_inp = x[t]
        new_attention = torch.zeros(B, U, dtype=x.dtype) if attention is None else attention[t].detach()   # :518
        for i, (scope, residual) in enumerate(cells):
            inp = torch.cat([cur_inp, new_attention], -1)          # :526
            nh, nc = lstm_cell(inp, hs[i], cs[i], w[scope + "/kernel"], w[scope + "/bias"], forget_bias)
            hs[i], cs[i] = nh, nc
            cur_inp = nh + inp[:, :U] if residual else nh          # gnmt_residual_fn :587-613: outputs + actual inputs
        outs.append(cur_inp)
    return torch.stack(outs)


def nmt_loss(outputs, proj_kernel, target_output, target_sequence_length, batch_size=None):
    """model.py:685-686 (logits = output_layer(rnn_output), a Dense without bias, :497-499) and _compute_loss :824-838.
    outputs [T,B,U]; target_output [B,T] ints (transposed at :827-828); returns (loss, logits [T,B,V])."""
    T, B, _ = outputs.shape
    logits = outputs @ proj_kernel
    labels = target_output.long().t()                               # [T,B]
    crossent = -torch.log_softmax(logits, -1).gather(-1, labels.unsqueeze(-1)).squeeze(-1)    # :820-821
    target_weights = (torch.arange(T).unsqueeze(0) < target_sequence_length.long().unsqueeze(1)).to(outputs.dtype).t()  # :833-836
    loss = (crossent * target_weights).sum() / float(batch_size if batch_size is not None else B)   # :837-838
    return loss, logits


# ---- decoder cell 0 with the attention wrapper: the first device's share of the decoder ----
# gnmt_model.py:309-325 (memory = encoder outputs, batch-major; normed Bahdanau attention over it with
# memory_sequence_length = source_sequence_length, attention_model.py:173-178), :366-374 (AttentionWrapper(cell 0,
# attention_layer_size=None, output_attention=False) inside GNMTAttentionMultiCell_1, zero initial state) and
# model.py:622-640 (embedding lookup of the time-major target_input, dynamic_decode with a TrainingHelper: a scan over
# the padded target steps).  AttentionWrapper and BahdanauAttention live in TensorFlow (un-vendored); their published
# algorithm is restated: values = memory with the steps past each source length zeroed, keys = values W_mem,
# cell input = concat([x_t, attention_{t-1}]), query = cell output h_t,
# score[b, j] = sum_u nv[u] tanh(keys[b, j, u] + (h_t W_q)[b, u] + attention_b[u]), nv = attention_g v / ||v||,
# score = -inf past the source length, alignments = softmax_j, attention_t = context = sum_j alignments values.
DA = "dynamic_seq2seq/decoder/"
EMB_DEC = DA + "embedding_decoder"
ATT_CELL = DA + "multi_rnn_cell_part1/cell_0_attention/attention/basic_lstm_cell"
ATT_MEM = DA + "memory_layer/kernel"
ATT_Q = DA + "multi_rnn_cell_part1/cell_0_attention/attention/bahdanau_attention/query_layer/kernel"
ATT_V = DA + "multi_rnn_cell_part1/cell_0_attention/attention/bahdanau_attention/attention_v"
ATT_G = DA + "multi_rnn_cell_part1/cell_0_attention/attention/bahdanau_attention/attention_g"
ATT_B = DA + "multi_rnn_cell_part1/cell_0_attention/attention/bahdanau_attention/attention_b"


def attention_cell_forward(target_input, memory, source_sequence_length, w, forget_bias=1.0):
    """target_input [B,T] ints; memory [S,B,U] (the encoder's time-major outputs); source_sequence_length [B] >= 1.
    Returns (cell outputs [T,B,U] = outputs_1.rnn_output, attention per step [T,B,U])."""
    emb = w[EMB_DEC][target_input.long().t()]                       # model.py:624-627
    mem = memory.transpose(0, 1)                                    # gnmt_model.py:309-312
    B, S, U = mem.shape
    mask = torch.arange(S).unsqueeze(0) < source_sequence_length.long().unsqueeze(1)       # [B,S]
    values = mem * mask.unsqueeze(-1).to(mem.dtype)
    keys = values @ w[ATT_MEM]
    v = w[ATT_V]
    nv = w[ATT_G] * v * torch.rsqrt((v * v).sum())
    h = torch.zeros(B, U, dtype=mem.dtype)
    c = torch.zeros(B, U, dtype=mem.dtype)
    att = torch.zeros(B, U, dtype=mem.dtype)
    outs, atts = [], []
    for t in range(emb.shape[0]):
        h, c = lstm_cell(torch.cat([emb[t], att], -1), h, c, w[ATT_CELL + "/kernel"], w[ATT_CELL + "/bias"], forget_bias)
        pq = h @ w[ATT_Q]
        score = (nv * torch.tanh(keys + pq.unsqueeze(1) + w[ATT_B])).sum(-1)
        score = torch.where(mask, score, torch.full_like(score, float("-inf")))
        align = torch.softmax(score, -1)
        att = (align.unsqueeze(-1) * values).sum(1)
        outs.append(h)
        atts.append(att)
    return torch.stack(outs), torch.stack(atts)
