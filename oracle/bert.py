"""CPU restatement of the reference's BERT stage slice. TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the bench's CPU-baseline leg may import this
module; the shipped stage never does.

Follows bert/models/bert/modeling_slice.py of the reference op for op, on
torch CPU tensors (fp64 for the checker, fp32 for the timed CPU baseline);
backward comes from torch.autograd, which is independent of the hand-derived
backward the HIP stage runs.

Pins (tests/test_oracle_bert.py): gelu vs torch's erf GELU and special values;
layer_norm vs torch.nn.functional.layer_norm and the zero-mean/unit-variance
invariant; attention vs a brute-force triple loop and vs
scaled_dot_product_attention; dense backward vs closed forms; the whole layer's
autograd vs central finite differences; parameter bytes vs the figures held in
profiling_results/bert-48-pbs-2.txt:3,5 of the reference.
What no reference fixture pins ("parity unpinned" by the reference's own tests,
which hold no numeric vector for this path): tf.contrib.layers.layer_norm's
epsilon (taken as 1e-12 inside the rsqrt, biased variance) and tf.erf's ULPs.
"""
import math

import torch


def gelu(x):
    """modeling_slice.py:30-43: x * 0.5 * (1 + erf(x / sqrt(2)))."""
    cdf = 0.5 * (1.0 + torch.erf(x / math.sqrt(2.0)))
    return x * cdf


def layer_norm(x, gamma, beta, eps=1e-12):
    """modeling_slice.py:152-155 -> tf.contrib.layers.layer_norm over the last axis:
    biased variance, eps inside the rsqrt, then gamma/beta."""
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    return (x - mean) * torch.rsqrt(var + eps) * gamma + beta


def dense(x, kernel, bias):
    """tf.layers.dense: x @ kernel[in,out] + bias."""
    return x @ kernel + bias


def attention_mask_from_input_mask(input_mask, from_seq):
    """modeling_slice.py:323-354: [B,T] 0/1 -> [B,F,T] float (ones column times to_mask)."""
    b, t = input_mask.shape
    return torch.ones(b, from_seq, 1, dtype=torch.float64) * input_mask.reshape(b, 1, t).to(torch.float64)


def attention_layer(x2d, w, prefix, batch, seq, heads, mask=None):
    """modeling_slice.py:357-549 (self-attention, 2-D in and out).

    x2d [B*S, H]; mask [B,S,S] of 0/1 or None (all ones: the adder vanishes)."""
    hidden = x2d.shape[1]
    d = hidden // heads
    q = dense(x2d, w[prefix + "query/kernel"], w[prefix + "query/bias"])
    k = dense(x2d, w[prefix + "key/kernel"], w[prefix + "key/bias"])
    v = dense(x2d, w[prefix + "value/kernel"], w[prefix + "value/bias"])

    def transpose_for_scores(t):                     # :427-433
        return t.reshape(batch, seq, heads, d).permute(0, 2, 1, 3)

    q, k, v = transpose_for_scores(q), transpose_for_scores(k), transpose_for_scores(v)
    scores = q @ k.transpose(-1, -2)                 # :499
    scores = scores * (1.0 / math.sqrt(float(d)))    # :500-501
    if mask is not None:                             # :503-514
        adder = (1.0 - mask.to(scores.dtype).unsqueeze(1)) * -10000.0
        scores = scores + adder
    probs = torch.softmax(scores, dim=-1)            # :518
    ctx = probs @ v                                  # :533
    ctx = ctx.permute(0, 2, 1, 3)                    # :536
    return ctx.reshape(batch * seq, hidden)          # :538-542


def encoder_layer(x2d, w, layer_idx, batch, seq, heads, mask=None):
    """modeling_slice.py:942-1001 with dropout 0."""
    p = "bert/encoder/layer_%d/" % layer_idx
    ctx = attention_layer(x2d, w, p + "attention/self/", batch, seq, heads, mask)
    attn = dense(ctx, w[p + "attention/output/dense/kernel"], w[p + "attention/output/dense/bias"])
    attn = layer_norm(attn + x2d, w[p + "attention/output/LayerNorm/gamma"],
                      w[p + "attention/output/LayerNorm/beta"])
    inter = gelu(dense(attn, w[p + "intermediate/dense/kernel"], w[p + "intermediate/dense/bias"]))
    out = dense(inter, w[p + "output/dense/kernel"], w[p + "output/dense/bias"])
    return layer_norm(out + attn, w[p + "output/LayerNorm/gamma"], w[p + "output/LayerNorm/beta"])


def embedding_stage(input_ids, token_type_ids, w):
    """modeling_slice.py:794-821 = embedding_lookup :170-217 + embedding_postprocessor
    :220-320 (gather; one-hot matmul for token types; first S position rows; LayerNorm)."""
    b, s = input_ids.shape
    word = w["bert/embeddings/word_embeddings"][input_ids.long()]
    type_table = w["bert/embeddings/token_type_embeddings"]
    one_hot = torch.nn.functional.one_hot(token_type_ids.long().reshape(-1), type_table.shape[0]).to(word.dtype)
    out = word + (one_hot @ type_table).reshape(b, s, -1)
    out = out + w["bert/embeddings/position_embeddings"][:s].reshape(1, s, -1)
    return layer_norm(out, w["bert/embeddings/LayerNorm/gamma"], w["bert/embeddings/LayerNorm/beta"])


def stage_forward(x, w, layers, batch, seq, heads, mask=None, token_type_ids=None):
    """One pipeline stage: optional embedding (when ``x`` holds ids) + reshape
    (:919-938) + the encoder layers in ``layers``.  Returns [B*S, H]."""
    if not x.dtype.is_floating_point:
        if token_type_ids is None:
            token_type_ids = torch.zeros_like(x)
        x = embedding_stage(x, token_type_ids, w).reshape(batch * seq, -1)
    for l in layers:
        x = encoder_layer(x, w, l, batch, seq, heads, mask)
    return x


def to_torch(weights, dtype=torch.float64, requires_grad=False):
    out = {}
    for k, v in weights.items():
        t = torch.as_tensor(v).to(dtype).clone()
        t.requires_grad_(requires_grad)
        out[k] = t
    return out


def stage_vjp(x, w, d_out, layers, batch, seq, heads, mask=None):
    """The reference's stage backward, tf.gradients(ys=out, xs=[x]+vars, grad_ys=d_out)
    (bert/graph.py:110-123): returns (out, d_x or None, {name: d_w})."""
    names = sorted(w)
    is_act = x.dtype.is_floating_point
    if is_act:
        x = x.clone().requires_grad_(True)
    out = stage_forward(x, w, layers, batch, seq, heads, mask)
    xs = ([x] if is_act else []) + [w[n] for n in names]
    grads = torch.autograd.grad(out, xs, grad_outputs=d_out, allow_unused=True)
    d_x = grads[0] if is_act else None
    d_w = {n: g for n, g in zip(names, grads[1 if is_act else 0:]) if g is not None}
    return out.detach(), d_x, d_w
