"""CPU restatement of the reference's GNMT encoder stage. TEST INFRASTRUCTURE ONLY.

Follows gnmt/nmt/gnmt_model.py:61-221 (DAPPLE branch: embedding lookup, one bidirectional
layer, uni layer 1 without residual, uni layers 2.. with residual) and
gnmt/nmt/model_helper.py:399-456 (_single_cell: BasicLSTMCell(num_units, forget_bias) +
ResidualWrapper).  BasicLSTMCell itself lives in TensorFlow (un-vendored); its published
algorithm is restated here: one kernel [in+U, 4U] applied to concat([x, h], 1), bias [4U],
gate order i, j, f, o, c' = c*sigmoid(f + forget_bias) + sigmoid(i)*tanh(j),
h' = tanh(c')*sigmoid(o).  tf.nn.dynamic_rnn with full-length sequences is a plain scan from a
zero state; the backward cell of bidirectional_dynamic_rnn scans the reversed sequence.

Pins (tests/test_oracle_gnmt.py): the cell vs torch.nn.LSTMCell after permuting the gate
blocks (torch order i, f, g, o) and folding forget_bias into the bias; the kernel layout
[in+U, 4U] vs the shape held by gnmt/nmt/model_test.py:86 ((10, 20) for in = U = 5); the
scan vs an explicit Python loop; the bidirectional layer vs torch.nn.LSTM(bidirectional=True).
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


def dynamic_rnn(x, kernel, bias, forget_bias=1.0, reverse=False):
    """x [T,B,I] time-major, zero initial state, all sequences full length -> outputs [T,B,U]."""
    T, B, _ = x.shape
    U = kernel.shape[1] // 4
    h = torch.zeros(B, U, dtype=x.dtype)
    c = torch.zeros(B, U, dtype=x.dtype)
    outs = [None] * T
    order = range(T - 1, -1, -1) if reverse else range(T)
    for t in order:
        h, c = lstm_cell(x[t], h, c, kernel, bias, forget_bias)
        outs[t] = h
    return torch.stack(outs)


def encoder_forward(ids, w, num_layers, forget_bias=1.0):
    """ids [B,T] int -> encoder outputs [T,B,U] (gnmt_model.py:78-210)."""
    emb = w[EMB][ids.long().t()]                      # time-major lookup (:78-79, :90-91)
    cells = cell_names(num_layers)
    fw = dynamic_rnn(emb, w[cells[0][0] + "/kernel"], w[cells[0][0] + "/bias"], forget_bias)
    bw = dynamic_rnn(emb, w[cells[1][0] + "/kernel"], w[cells[1][0] + "/bias"], forget_bias, reverse=True)
    x = torch.cat([fw, bw], -1)                       # :108
    for scope, _, residual in cells[2:]:
        y = dynamic_rnn(x, w[scope + "/kernel"], w[scope + "/bias"], forget_bias)
        x = y + x if residual else y                  # ResidualWrapper, model_helper.py:445-448
    return x


def to_torch(weights, dtype=torch.float64, requires_grad=False):
    return {k: torch.as_tensor(v).to(dtype).clone().requires_grad_(requires_grad) for k, v in weights.items()}


def stage_vjp(ids, w, d_out, num_layers, forget_bias=1.0):
    names = sorted(w)
    out = encoder_forward(ids, w, num_layers, forget_bias)
    grads = torch.autograd.grad(out, [w[n] for n in names], grad_outputs=d_out, allow_unused=True)
    return out.detach(), None, {n: g for n, g in zip(names, grads) if g is not None}
