"""CPU restatement of the SQuAD output layer of the last BERT stage. TEST INFRASTRUCTURE ONLY.

bert/models/bert/bert.py:669-718 (build_output_layer_squad), line by line in torch so that autograd gives the
gradients.  Pins (tests/test_oracle_head.py): compute_loss equals torch.nn.functional.cross_entropy (mean
reduction) on in-range positions; brute-force loops on a tiny case; positions outside [0, seq) follow
tf.one_hot (an all-zero row: no loss term).

classification_loss restates pooler_stage (bert/models/bert/modeling_slice.py:849-868) and
build_output_layer_classification (bert/models/bert/bert.py:642-664).  Pins: the cross entropy equals
torch.nn.functional.cross_entropy; tf.contrib.layers.l2_regularizer(scale)(w) is scale * tf.nn.l2_loss(w) =
scale * sum(w^2) / 2 (TensorFlow's published definition, un-vendored), checked through its gradient scale * w;
a brute-force loop on a tiny case.

xlnet_squad_loss restates XLnetLoss.call (xlnet/losses/xlnet_loss.py:36-120), the SQuAD-2 head of the last XLNet
stage.  Pins: the masked log-softmax terms equal torch.nn.functional.cross_entropy on the masked logits; the layer
normalisation equals torch.nn.functional.layer_norm (eps 1e-14); the answerability term equals
torch.nn.functional.binary_cross_entropy_with_logits; the one-hot einsums equal plain row picks; a brute-force loop
on a tiny case.  The reference draws the dropout at :103 from TensorFlow's generator: the factor is an input here.
"""
import torch


def squad_loss(final_hidden, output_weights, output_bias, start_positions, end_positions):
    """final_hidden [batch, seq, hidden]; returns (loss, start_logits [batch, seq], end_logits [batch, seq])."""
    batch_size, seq_length, hidden_size = final_hidden.shape                         # :672-675
    final_hidden_matrix = final_hidden.reshape(batch_size * seq_length, hidden_size)  # :685-686
    logits = final_hidden_matrix @ output_weights.t()                                # :687 (transpose_b=True)
    logits = logits + output_bias                                                    # :688
    logits = logits.reshape(batch_size, seq_length, 2).permute(2, 0, 1)              # :690-691
    start_logits, end_logits = logits[0], logits[1]                                  # :693-695

    def compute_loss(lg, positions):                                                 # :699-705
        pos = positions.long()
        valid = (pos >= 0) & (pos < seq_length)
        one_hot = torch.zeros_like(lg)
        one_hot[valid, pos[valid]] = 1.0
        log_probs = torch.log_softmax(lg, dim=-1)
        return -torch.mean(torch.sum(one_hot * log_probs, dim=-1))

    loss = (compute_loss(start_logits, start_positions) + compute_loss(end_logits, end_positions)) / 2.0   # :707-714
    return loss, start_logits, end_logits


def classification_loss(sequence_output, pooler_kernel, pooler_bias, fc_weights, fc_biases, labels, l2_scale=1e-3):
    """sequence_output [batch, seq, hidden]; returns (loss, logits [batch, num_labels], pooled [batch, hidden])."""
    first_token_tensor = sequence_output[:, 0, :]                                    # modeling_slice.py:861
    pooled = torch.tanh(first_token_tensor @ pooler_kernel + pooler_bias)            # :862-866
    logits = pooled @ fc_weights + fc_biases                                         # bert.py:644-652
    log_probs = torch.log_softmax(logits, dim=-1)
    ce = -log_probs[torch.arange(logits.shape[0]), labels.long()]                    # :656-657
    loss = ce.mean() + l2_scale * 0.5 * (fc_weights ** 2).sum()                      # :655-659, l2_regularizer(1e-3)
    return loss, logits, pooled


def regression_loss(sequence_output, pooler_kernel, pooler_bias, fc_weights, fc_biases, labels, l2_scale=1e-3):
    """build_output_layer_regression, bert/models/bert/bert.py:615-640, behind pooler_stage.  sequence_output
    [batch, seq, hidden], fc_weights [hidden, 1], labels float [batch] (the placeholder's shape,
    bert_finetune.py:212).  Returns (loss, prediction [batch, 1], pooled)."""
    first_token_tensor = sequence_output[:, 0, :]                                    # modeling_slice.py:861
    pooled = torch.tanh(first_token_tensor @ pooler_kernel + pooler_bias)            # :862-866
    prediction = pooled @ fc_weights + fc_biases                                     # bert.py:617-625, [batch, 1]
    # :628-631: [batch, 1] - [batch] broadcasts to [batch, batch]; reduce_mean runs over all of it
    loss = ((prediction - labels) ** 2).mean() + l2_scale * 0.5 * (fc_weights ** 2).sum()
    return loss, prediction, pooled


def xlnet_squad_loss(output, w, cls_index, start_positions, end_positions, is_impossible, p_mask, dropout_mask=None):
    """XLnetLoss.call, xlnet/losses/xlnet_loss.py:36-120, line by line.

    output [seq, batch, d_model] (the last stage's content stream after slice_xlnet.py:236); w: dict with
      start_w [d_model, 1], start_b [1]                      self.dense          (:19)
      end_w0 [2*d_model, d_model], end_b0 [d_model]          self.dense_0        (:20-23)
      ln_gamma, ln_beta [d_model]                            self.layer_norm     (:24; eps = K.epsilon()**2 = 1e-14)
      end_w1 [d_model, 1], end_b1 [1]                        self.dense_1        (:25)
      ans_w0 [2*d_model, d_model], ans_b0 [d_model]          self.dense_0_1      (:26-29)
      ans_w1 [d_model, 1]                                    self.dense_1_1      (:30-34, no bias)
    cls_index, start_positions, end_positions: integer [batch]; is_impossible: float [batch]; p_mask float [batch, seq].
    dropout_mask [batch, d_model] stands for keras.layers.Dropout(rate=0.1)(., training=True) at :103: the factor each
    element is multiplied by (0 or 1/0.9 in the reference, drawn by TensorFlow's generator); None = all ones.
    Returns (total_loss, start_logits [batch, seq], end_logits [batch, seq], cls_logits [batch])."""
    seq = output.shape[0]

    def one_hot(idx):                                                                # tf.one_hot: all-zero row outside [0, seq)
        idx = idx.long()
        valid = (idx >= 0) & (idx < seq)
        oh = torch.zeros(idx.shape[0], seq, dtype=output.dtype)
        oh[valid, idx[valid]] = 1.0
        return oh

    def layer_norm(x):                                                               # layers/layer_normalization.py:69-78
        mean = x.mean(dim=-1, keepdim=True)
        variance = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
        std = torch.sqrt(variance + 1e-7 * 1e-7)
        return (x - mean) / std * w["ln_gamma"] + w["ln_beta"]

    start_logits = output @ w["start_w"] + w["start_b"]                              # :51
    start_logits = start_logits.squeeze(-1).t()                                      # :52  [batch, seq]
    start_logits_masked = start_logits * (1 - p_mask) - 1e30 * p_mask                # :53
    start_log_probs = torch.log_softmax(start_logits_masked, dim=-1)                 # :54

    start_index = one_hot(start_positions)                                           # :59-61
    start_features = torch.einsum("lbh,bl->bh", output, start_index)                 # :64
    start_features = start_features.unsqueeze(0).repeat(seq, 1, 1)                   # :65-66
    tmp_concat = torch.cat([output, start_features], dim=-1)                         # :67
    end_logits = torch.tanh(tmp_concat @ w["end_w0"] + w["end_b0"])                  # :68
    end_logits = layer_norm(end_logits)                                              # :70
    end_logits = end_logits @ w["end_w1"] + w["end_b1"]                              # :72
    end_logits = end_logits.squeeze(-1).t()                                          # :73
    end_logits_masked = end_logits * (1 - p_mask) - 1e30 * p_mask                    # :74
    end_log_probs = torch.log_softmax(end_logits_masked, dim=-1)                     # :76

    start_loss = (-(start_log_probs * start_index).sum(dim=-1)).mean()               # :78-79
    end_index = one_hot(end_positions)                                               # :82-84
    end_loss = (-(end_log_probs * end_index).sum(dim=-1)).mean()                     # :86-87
    total_loss = (start_loss + end_loss) * 0.5                                       # :88

    cls_one_hot = one_hot(cls_index)                                                 # :91-95
    cls_feature = torch.einsum("lbh,bl->bh", output, cls_one_hot)                    # :98
    start_p = torch.softmax(start_logits_masked, dim=-1)                             # :100
    start_feature = torch.einsum("lbh,bl->bh", output, start_p)                      # :102-103
    ans_feature = torch.cat([start_feature, cls_feature], dim=-1)                    # :106
    ans_feature = torch.tanh(ans_feature @ w["ans_w0"] + w["ans_b0"])                # :107
    if dropout_mask is not None:
        ans_feature = ans_feature * dropout_mask                                     # :108
    cls_logits = (ans_feature @ w["ans_w1"]).squeeze(-1)                             # :109-110

    labels = is_impossible.reshape(-1)                                               # :112
    # tf.nn.sigmoid_cross_entropy_with_logits: max(x, 0) - x z + log(1 + exp(-|x|))
    regression_loss = torch.clamp(cls_logits, min=0) - cls_logits * labels + torch.log1p(torch.exp(-cls_logits.abs()))  # :113-116
    total_loss = total_loss + regression_loss.mean() * 0.5                           # :117-118
    return total_loss, start_logits, end_logits, cls_logits
