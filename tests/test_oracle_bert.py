"""Pins the BERT oracle against independent routines, closed forms and brute force.

The reference's own tests hold no numeric vector for the stage path
(bert/models/bert/modeling_test.py:114-124 checks shapes only), so each function
is pinned by something a plausible mistake would break.
"""
import math

import numpy as np
import pytest
import torch

from dapple_amd import synthetic
from oracle import bert as ob

torch.manual_seed(0)
D = torch.float64


def test_gelu_matches_erf_form_and_special_values():
    x = torch.linspace(-6, 6, 1001, dtype=D)
    assert torch.allclose(ob.gelu(x), torch.nn.functional.gelu(x, approximate="none"), atol=1e-14)
    assert ob.gelu(torch.zeros(1, dtype=D)).item() == 0.0
    x0 = torch.zeros(1, dtype=D, requires_grad=True)
    (g,) = torch.autograd.grad(ob.gelu(x0).sum(), x0)
    assert abs(g.item() - 0.5) < 1e-15
    # the tanh approximation differs by ~1e-3: the erf form is the one in use
    assert (ob.gelu(x) - torch.nn.functional.gelu(x, approximate="tanh")).abs().max() > 1e-4


def test_layer_norm_matches_torch_and_invariants():
    x = torch.randn(7, 64, dtype=D) * 3 + 1.5
    g = torch.randn(64, dtype=D)
    b = torch.randn(64, dtype=D)
    ref = torch.nn.functional.layer_norm(x, (64,), g, b, eps=1e-12)
    assert torch.allclose(ob.layer_norm(x, g, b), ref, atol=1e-12)
    y = ob.layer_norm(x, torch.ones(64, dtype=D), torch.zeros(64, dtype=D))
    assert y.mean(-1).abs().max() < 1e-12
    assert (y.var(-1, unbiased=False) - 1).abs().max() < 1e-9
    # with gamma == 1 the input gradient of every row sums to zero
    xr = x.clone().requires_grad_(True)
    out = ob.layer_norm(xr, torch.ones(64, dtype=D), torch.zeros(64, dtype=D))
    (dx,) = torch.autograd.grad(out, xr, torch.randn_like(out))
    assert dx.sum(-1).abs().max() < 1e-10


def _brute_attention(x, w, p, B, S, N, mask):
    H = x.shape[1]
    d = H // N
    q = x @ w[p + "query/kernel"] + w[p + "query/bias"]
    k = x @ w[p + "key/kernel"] + w[p + "key/bias"]
    v = x @ w[p + "value/kernel"] + w[p + "value/bias"]
    out = np.zeros((B * S, H))
    for b in range(B):
        for n in range(N):
            for i in range(S):
                s = np.zeros(S)
                for j in range(S):
                    s[j] = np.dot(q[b * S + i, n * d:(n + 1) * d], k[b * S + j, n * d:(n + 1) * d]) / math.sqrt(d)
                    if mask is not None:
                        s[j] += (1.0 - mask[b, i, j]) * -10000.0
                e = np.exp(s - s.max())
                pr = e / e.sum()
                for j in range(S):
                    out[b * S + i, n * d:(n + 1) * d] += pr[j] * v[b * S + j, n * d:(n + 1) * d]
    return out


@pytest.mark.parametrize("use_mask", [False, True])
def test_attention_vs_brute_force_and_sdpa(use_mask):
    B, S, N, d = 2, 5, 2, 3
    H = N * d
    w = synthetic.bert_weights(7, 1, H, 4 * H, stddev=0.5, perturb=True)
    wt = ob.to_torch(w)
    x = torch.randn(B * S, H, dtype=D)
    mask = None
    if use_mask:
        im = torch.tensor([[1, 1, 1, 0, 0], [1, 1, 1, 1, 0]])
        mask = ob.attention_mask_from_input_mask(im, S)
        assert mask.shape == (B, S, S) and mask[0, 2].tolist() == [1, 1, 1, 0, 0]
    p = "bert/encoder/layer_0/attention/self/"
    got = ob.attention_layer(x, wt, p, B, S, N, mask)
    want = _brute_attention(x.numpy(), {k: v.numpy() for k, v in wt.items()}, p, B, S, N,
                            None if mask is None else mask.numpy())
    assert np.allclose(got.numpy(), want, atol=1e-12)
    # library routine: scaled_dot_product_attention with an additive mask
    q = (x @ wt[p + "query/kernel"] + wt[p + "query/bias"]).reshape(B, S, N, d).transpose(1, 2)
    k = (x @ wt[p + "key/kernel"] + wt[p + "key/bias"]).reshape(B, S, N, d).transpose(1, 2)
    v = (x @ wt[p + "value/kernel"] + wt[p + "value/bias"]).reshape(B, S, N, d).transpose(1, 2)
    add = None if mask is None else ((1.0 - mask) * -10000.0).unsqueeze(1)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=add)
    assert torch.allclose(got, ref.transpose(1, 2).reshape(B * S, H), atol=1e-12)


def test_all_ones_mask_is_identity():
    B, S, N, H = 2, 4, 2, 8
    wt = ob.to_torch(synthetic.bert_weights(3, 1, H, 16, stddev=0.3, perturb=True))
    x = torch.randn(B * S, H, dtype=D)
    ones = ob.attention_mask_from_input_mask(torch.ones(B, S, dtype=torch.int32), S)
    a = ob.encoder_layer(x, wt, 0, B, S, N, None)
    b = ob.encoder_layer(x, wt, 0, B, S, N, ones)
    assert torch.equal(a, b)


def test_dense_backward_closed_forms():
    x = torch.randn(6, 5, dtype=D, requires_grad=True)
    k = torch.randn(5, 4, dtype=D, requires_grad=True)
    b = torch.randn(4, dtype=D, requires_grad=True)
    dy = torch.randn(6, 4, dtype=D)
    dx, dk, db = torch.autograd.grad(ob.dense(x, k, b), [x, k, b], dy)
    assert torch.allclose(dx, dy @ k.T) and torch.allclose(dk, x.T @ dy) and torch.allclose(db, dy.sum(0))


def test_layer_vjp_vs_finite_differences():
    B, S, N, H, F = 1, 3, 2, 4, 8
    w = ob.to_torch(synthetic.bert_weights(11, 1, H, F, stddev=0.4, perturb=True), requires_grad=True)
    x = torch.randn(B * S, H, dtype=D)
    dy = torch.randn(B * S, H, dtype=D)
    out, dx, dw = ob.stage_vjp(x, w, dy, [0], B, S, N)
    eps = 1e-6

    def f(xx, ww):
        return (ob.stage_forward(xx, ww, [0], B, S, N) * dy).sum().item()

    for idx in [(0, 0), (2, 3), (1, 2)]:
        xp, xm = x.clone(), x.clone()
        xp[idx] += eps
        xm[idx] -= eps
        assert abs((f(xp, w) - f(xm, w)) / (2 * eps) - dx[idx].item()) < 1e-6
    for name in w:
        wd = {k: v.detach().clone() for k, v in w.items()}
        flat = wd[name].view(-1)
        i = flat.numel() // 2
        flat[i] += eps
        fp = f(x, wd)
        flat[i] -= 2 * eps
        fm = f(x, wd)
        assert abs((fp - fm) / (2 * eps) - dw[name].reshape(-1)[i].item()) < 1e-6, name


def test_embedding_stage_brute_force_and_scatter():
    V, T, P, H, B, S = 11, 2, 8, 6, 2, 4
    w = ob.to_torch(synthetic.bert_weights(5, 0, H, 8, embeddings=(V, T, P), stddev=0.5, perturb=True),
                    requires_grad=True)
    ids = torch.tensor([[3, 3, 7, 0], [10, 3, 1, 1]], dtype=torch.int32)
    tt = torch.tensor([[0, 0, 1, 1], [0, 1, 0, 1]], dtype=torch.int32)
    got = ob.embedding_stage(ids, tt, w)
    for b in range(B):
        for s in range(S):
            row = (w["bert/embeddings/word_embeddings"][ids[b, s]] + w["bert/embeddings/token_type_embeddings"][tt[b, s]]
                   + w["bert/embeddings/position_embeddings"][s])
            want = ob.layer_norm(row, w["bert/embeddings/LayerNorm/gamma"], w["bert/embeddings/LayerNorm/beta"])
            assert torch.allclose(got[b, s], want, atol=1e-12)
    (dword,) = torch.autograd.grad(got.sum() + (got ** 2).sum(), w["bert/embeddings/word_embeddings"])
    used = {3, 7, 0, 10, 1}
    for v in range(V):
        assert (dword[v].abs().sum() > 0) == (v in used)


def test_parameter_bytes_match_reference_profile():
    # profiling_results/bert-48-pbs-2.txt:5 parameter_size=50384896 per encoder layer,
    # :3 127131648 for the embeddings (type vocab 2), fp32
    per_layer = sum(int(np.prod(s)) for _, s in synthetic.bert_layer_shapes(1024, 4096))
    assert per_layer * 4 == 50384896
    emb = sum(int(np.prod(s)) for _, s in synthetic.bert_embedding_shapes(30522, 1024, 2, 512))
    assert emb * 4 == 127131648


def test_output_shapes_like_reference_modeling_test():
    # modeling_test.py:114-124 pins shapes: sequence output [B,S,H]
    B, S, N, H = 2, 7, 4, 32
    w = ob.to_torch(synthetic.bert_weights(1, 2, H, 37, embeddings=(99, 16, 512)))
    ids = torch.randint(0, 99, (B, S), dtype=torch.int32)
    out = ob.stage_forward(ids, w, [0, 1], B, S, N)
    assert out.shape == (B * S, H)
