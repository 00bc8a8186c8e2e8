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
