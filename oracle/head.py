"""CPU restatement of the SQuAD output layer of the last BERT stage. TEST INFRASTRUCTURE ONLY.

bert/models/bert/bert.py:669-718 (build_output_layer_squad), line by line in torch so that autograd gives the
gradients.  Pins (tests/test_oracle_head.py): compute_loss equals torch.nn.functional.cross_entropy (mean
reduction) on in-range positions; brute-force loops on a tiny case; positions outside [0, seq) follow
tf.one_hot (an all-zero row: no loss term).
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
