"""CPU restatement of the reference's XLNet stage layers. TEST INFRASTRUCTURE ONLY.

Restates xlnet/layers/rel_multihead_attn.py:71-149 (the einsums of _rel_attn_core and call),
lambda_funcs.py:7-44 (attention mask), :50-79 (position embedding), :85-93 (rel_shift),
segment_embed.py:33-54 (segment matrix), position_wise_feed_forward.py:92-105,
layer_normalization.py:69-78 (epsilon = K.epsilon()**2 = 1e-14), activations/gelu.py:6-11 (tanh
form) and the layer body models/slice_xlnet.py:164-180 (attention -> add -> LN -> FFN -> add -> LN).

The reference implements the content stream only, with memory length hard-wired to 0
(lambda_funcs.py:20,36; segment_embed.py:37).  What BASELINE configs[4] adds - memory of length
mlen (keys/values from concat(mem, h), positions running from klen down to -qlen), a query stream
g that shares k, v and all weights, and permutation masks - follows the XLNet formulation
(Yang et al. 2019, section 2.3-2.5; the reference's commented einsums are that code) and is
"parity unpinned" by the reference: it is pinned by a brute-force loop implementation and by
reducing to the reference form at mlen = 0 / one stream (tests/test_oracle_xlnet.py).
"""
import math

import torch


def gelu_tanh(x):
    """activations/gelu.py:6-11."""
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x * x * x)))


def layer_norm(x, gamma, beta, eps=1e-14):
    """layer_normalization.py:69-78."""
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * gamma + beta


def rel_shift(x, klen):
    """lambda_funcs.py:85-93, op for op."""
    s = x.shape
    x = x.reshape(s[1], s[0], s[2], s[3])
    x = x[1:]
    x = x.reshape(s[0], s[1] - 1, s[2], s[3])
    return x[:, :klen]


def pos_emb(qlen, klen, d_model, bsz, dtype=torch.float64):
    """lambda_funcs.py:50-79 with beg = klen (the reference has klen == qlen): positions klen .. -qlen+1."""
    freq_seq = torch.arange(0, d_model, 2.0, dtype=dtype)
    inv_freq = 1 / (10000 ** (freq_seq / d_model))
    pos_seq = torch.arange(klen, -qlen, -1.0, dtype=dtype)
    sinusoid = torch.einsum("i,d->id", pos_seq, inv_freq)
    pe = torch.cat([torch.sin(sinusoid), torch.cos(sinusoid)], -1)
    return pe[:, None, :].repeat(1, bsz, 1)


def attn_mask_from_input_mask(input_mask, mlen=0):
    """lambda_funcs.py:7-44: input_mask [B, qlen] (1 = padding) -> [qlen, klen, B] of 0/1 (1 = masked);
    a key is masked where it is padding, except on the diagonal; memory is never masked."""
    b, qlen = input_mask.shape
    data_mask = input_mask.t()[None].to(torch.float64)                     # [1, qlen, B]
    data_mask = torch.cat([torch.zeros(1, mlen, b, dtype=torch.float64), data_mask], 1)
    attn_mask = (data_mask > 0).to(torch.float64)                           # [1, klen, B]
    non_tgt = torch.cat([torch.zeros(qlen, mlen, dtype=torch.float64), -torch.eye(qlen, dtype=torch.float64)], -1)
    return ((attn_mask + non_tgt[:, :, None]) > 0).to(torch.float64)        # [qlen, klen, B]


def seg_mat_from_ids(seg_ids, mlen=0):
    """segment_embed.py:33-54: seg_ids [qlen, B] -> 0/1 [qlen, klen, B] (1 = different segment)."""
    cat_ids = torch.cat([torch.zeros(mlen, seg_ids.shape[1], dtype=seg_ids.dtype), seg_ids], 0)
    return (seg_ids[:, None] != cat_ids[None, :]).to(torch.int64)


def rel_attn_core(q_head, k_head_h, v_head_h, k_head_r, seg_embed, seg_mat, r_w, r_r, r_s, attn_mask, scale):
    """rel_multihead_attn.py:71-115; seg_mat is the 0/1 index form of the one-hot matrix, attn_mask [q,k,B]."""
    klen = k_head_h.shape[0]
    ac = torch.einsum("ibnd,jbnd->ijbn", q_head + r_w, k_head_h)
    bd = rel_shift(torch.einsum("ibnd,jbnd->ijbn", q_head + r_r, k_head_r), klen)
    ef = torch.einsum("ibnd,snd->ibns", q_head + r_s, seg_embed)
    one_hot = torch.nn.functional.one_hot(seg_mat, 2).to(ef.dtype)         # [q,k,B,2]
    ef = torch.einsum("ijbs,ibns->ijbn", one_hot, ef)
    score = (ac + bd + ef) * scale - 1e30 * attn_mask[:, :, :, None].to(ac.dtype)
    prob = torch.softmax(score, 1)
    return torch.einsum("ijbn,jbnd->ibnd", prob, v_head_h)


def layer(streams, mem, w, l, heads, masks, seg_mat, pe):
    """One XLNet layer on one or two streams.  streams = [h] or [h, g], each [qlen, B, H]; mem [mlen,B,H] or
    None; masks = per-stream [qlen, klen, B]; keys/values always come from concat(mem, h)."""
    h = streams[0]
    H = h.shape[-1]
    d = H // heads
    p = "layer_%d/" % l
    wq, wk, wv, wr, wo = (w[p + n].reshape(H, heads, d) for n in ("q", "k", "v", "r", "o"))
    cat = h if mem is None or mem.shape[0] == 0 else torch.cat([mem, h], 0)
    k_head_h = torch.einsum("ibh,hnd->ibnd", cat, wk)
    v_head_h = torch.einsum("ibh,hnd->ibnd", cat, wv)
    k_head_r = torch.einsum("ibh,hnd->ibnd", pe, wr)
    seg_embed = w[p + "seg_emb"].reshape(2, heads, d)
    r_w, r_r, r_s = (w[p + n].reshape(heads, d) for n in ("bias_context", "bias_relative", "bias_segment"))
    outs = []
    for x, mask in zip(streams, masks):
        q_head = torch.einsum("ibh,hnd->ibnd", x, wq)
        vec = rel_attn_core(q_head, k_head_h, v_head_h, k_head_r, seg_embed, seg_mat, r_w, r_r, r_s, mask, 1 / d ** 0.5)
        attn_out = torch.einsum("ibnd,hnd->ibh", vec, wo)
        y = layer_norm(x + attn_out, w[p + "attn_ln/gamma"], w[p + "attn_ln/beta"])
        ff = gelu_tanh(y @ w[p + "ff/W1"] + w[p + "ff/b1"]) @ w[p + "ff/W2"] + w[p + "ff/b2"]
        outs.append(layer_norm(y + ff, w[p + "ff_ln/gamma"], w[p + "ff_ln/beta"]))
    return outs


def stage_forward(streams, mems, w, layers, heads, masks, seg_ids):
    """streams [h] / [h, g]; mems [L][mlen,B,H] or None; masks per stream; seg_ids [qlen,B] ints."""
    qlen, bsz, H = streams[0].shape
    mlen = 0 if mems is None else mems[0].shape[0]
    klen = mlen + qlen
    pe = pos_emb(qlen, klen, H, bsz, streams[0].dtype)
    seg_mat = seg_mat_from_ids(seg_ids, mlen)
    for idx, l in enumerate(layers):
        streams = layer(streams, None if mems is None else mems[idx], w, l, heads, masks, seg_mat, pe)
    return streams


def to_torch(weights, dtype=torch.float64, requires_grad=False):
    return {k: torch.as_tensor(v).to(dtype).clone().requires_grad_(requires_grad) for k, v in weights.items()}


def stage_vjp(streams, mems, w, d_outs, layers, heads, masks, seg_ids):
    names = sorted(w)
    xs = [s.clone().requires_grad_(True) for s in streams]
    outs = stage_forward(xs, mems, w, layers, heads, masks, seg_ids)
    grads = torch.autograd.grad(outs, xs + [w[n] for n in names], grad_outputs=list(d_outs), allow_unused=True)
    ns = len(xs)
    return [o.detach() for o in outs], list(grads[:ns]), {n: g for n, g in zip(names, grads[ns:]) if g is not None}


# ---- brute force (tiny sizes): scores from scalar loops, the relative position looked up directly ----
def brute_force_attention(x, cat, w, l, heads, mask, seg_ids_q, seg_ids_k, mlen):
    """attn_vec [qlen,B,N,D] for queries x against keys cat with position (mlen + i) - j."""
    qlen, bsz, H = x.shape
    klen = cat.shape[0]
    d = H // heads
    p = "layer_%d/" % l
    wq, wk, wv, wr = (w[p + n].reshape(H, heads, d) for n in ("q", "k", "v", "r"))
    seg = w[p + "seg_emb"].reshape(2, heads, d)
    r_w, r_r, r_s = (w[p + n].reshape(heads, d) for n in ("bias_context", "bias_relative", "bias_segment"))
    inv_freq = [1 / (10000 ** (2.0 * t / H)) for t in range(H // 2)]
    out = torch.zeros(qlen, bsz, heads, d, dtype=x.dtype)
    for b in range(bsz):
        for n in range(heads):
            for i in range(qlen):
                q = x[i, b] @ wq[:, n]
                sc = torch.zeros(klen, dtype=x.dtype)
                for j in range(klen):
                    k = cat[j, b] @ wk[:, n]
                    rel = float(mlen + i - j)
                    pe = torch.tensor([math.sin(rel * f) for f in inv_freq] + [math.cos(rel * f) for f in inv_freq], dtype=x.dtype)
                    kr = pe @ wr[:, n]
                    s = 1 if seg_ids_q[i, b] != seg_ids_k[j, b] else 0
                    sc[j] = ((q + r_w[n]) @ k + (q + r_r[n]) @ kr + (q + r_s[n]) @ seg[s, n]) / d ** 0.5 - 1e30 * mask[i, j, b]
                pr = torch.softmax(sc, 0)
                for j in range(klen):
                    out[i, b, n] += pr[j] * (cat[j, b] @ wv[:, n])
    return out
