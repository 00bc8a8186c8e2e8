"""Pins the XLNet oracle: rel_shift / position embedding / masks by brute force and truth tables, the
whole relative attention (incl. memory and the query stream) against scalar loops."""
import math

import numpy as np
import torch

from dapple_amd import synthetic
from oracle import xlnet as ox

D = torch.float64


def test_rel_shift_is_the_index_map_j_plus_qlen_minus_i():
    for qlen, klen in ((3, 3), (3, 5), (4, 6)):
        rlen = qlen + klen
        x = torch.arange(qlen * rlen * 2, dtype=D).reshape(qlen, rlen, 1, 2)
        y = ox.rel_shift(x, klen)
        assert y.shape == (qlen, klen, 1, 2)
        for i in range(qlen):
            for j in range(klen):
                assert torch.equal(y[i, j], x[i, j + qlen - i])


def test_pos_emb_direct_formula_and_reference_range():
    qlen, klen, d = 3, 5, 8
    pe = ox.pos_emb(qlen, klen, d, 2)
    assert pe.shape == (qlen + klen, 2, d)
    for r in range(qlen + klen):
        pos = klen - r
        for t in range(d // 2):
            f = 1 / (10000 ** (2.0 * t / d))
            assert abs(pe[r, 1, t].item() - math.sin(pos * f)) < 1e-12
            assert abs(pe[r, 0, d // 2 + t].item() - math.cos(pos * f)) < 1e-12
    # the reference's own range (klen == qlen): tf.range(qlen, -qlen, -1), 2*qlen entries (lambda_funcs.py:59-62)
    assert ox.pos_emb(4, 4, 8, 1).shape[0] == 8


def test_attn_mask_truth_table():
    im = torch.tensor([[0, 0, 1, 1], [0, 0, 0, 0]])          # batch 0: last two tokens are padding
    m = ox.attn_mask_from_input_mask(im)
    assert m.shape == (4, 4, 2)
    assert m[:, :, 1].sum() == 0
    want0 = torch.tensor([[0, 0, 1, 1], [0, 0, 1, 1], [0, 0, 0, 1], [0, 0, 1, 0]], dtype=D)   # diagonal exempt
    assert torch.equal(m[:, :, 0], want0)
    m2 = ox.attn_mask_from_input_mask(im, mlen=2)
    assert m2.shape == (4, 6, 2) and m2[:, :2].sum() == 0 and torch.equal(m2[:, 2:, 0], want0)


def test_seg_mat_and_perm_masks():
    seg = torch.tensor([[0], [0], [1]])
    sm = ox.seg_mat_from_ids(seg, mlen=1)
    assert sm[:, :, 0].tolist() == [[0, 0, 0, 1], [0, 0, 0, 1], [1, 1, 1, 0]]
    mh, mg = synthetic.xlnet_perm_masks(3, 6, 2, 2)
    assert mh.shape == (6, 8, 2) and mh[:, :2].sum() == 0 and mg[:, :2].sum() == 0
    for b in range(2):
        assert np.all(np.diagonal(mh[:, 2:, b]) == 0) and np.all(np.diagonal(mg[:, 2:, b]) == 1)
        # every pair (i, j), i != j, is visible in exactly one direction; the query mask adds only the diagonal
        assert np.all((mh[:, 2:, b] + mh[:, 2:, b].T)[~np.eye(6, dtype=bool)] == 1)
        assert np.all(mg[:, 2:, b] - mh[:, 2:, b] == np.eye(6))


def _tiny(mlen, streams):
    qlen, B, H, N, F = 3, 2, 8, 2, 16
    w = ox.to_torch(synthetic.xlnet_weights(5, 1, H, N, F, stddev=0.5, perturb=True))
    xs = [torch.randn(qlen, B, H, dtype=D) for _ in range(streams)]
    mem = torch.randn(mlen, B, H, dtype=D)
    seg = torch.tensor([[0, 1], [0, 1], [1, 1]])
    mh, mg = synthetic.xlnet_perm_masks(9, qlen, mlen, B)
    masks = [torch.tensor(mh, dtype=D), torch.tensor(mg, dtype=D)][:streams]
    return qlen, B, H, N, w, xs, mem, seg, masks


def test_attention_with_memory_and_query_stream_vs_brute_force():
    mlen = 2
    qlen, B, H, N, w, xs, mem, seg, masks = _tiny(mlen, 2)
    cat = torch.cat([mem, xs[0]], 0)
    seg_k = torch.cat([torch.zeros(mlen, B, dtype=seg.dtype), seg], 0)
    pe = ox.pos_emb(qlen, mlen + qlen, H, B)
    d = H // N
    p = "layer_0/"
    wq, wk, wv, wr = (w[p + n].reshape(H, N, d) for n in "qkvr")
    k_h = torch.einsum("ibh,hnd->ibnd", cat, wk)
    v_h = torch.einsum("ibh,hnd->ibnd", cat, wv)
    k_r = torch.einsum("ibh,hnd->ibnd", pe, wr)
    for x, mask in zip(xs, masks):
        got = ox.rel_attn_core(torch.einsum("ibh,hnd->ibnd", x, wq), k_h, v_h, k_r, w[p + "seg_emb"].reshape(2, N, d),
                               ox.seg_mat_from_ids(seg, mlen), w[p + "bias_context"].reshape(N, d),
                               w[p + "bias_relative"].reshape(N, d), w[p + "bias_segment"].reshape(N, d), mask, 1 / d ** 0.5)
        want = ox.brute_force_attention(x, cat, w, 0, N, mask, seg, seg_k, mlen)
        assert torch.allclose(got, want, atol=1e-10)


def test_one_stream_without_memory_is_the_reference_form():
    qlen, B, H, N, w, xs, mem, seg, masks = _tiny(0, 1)
    im = torch.tensor([[0, 0, 1], [0, 0, 0]])
    mask = ox.attn_mask_from_input_mask(im)
    (out,) = ox.stage_forward(xs, None, w, [0], N, [mask], seg)
    (out2,) = ox.stage_forward(xs, [torch.zeros(0, B, H, dtype=D)], w, [0], N, [mask], seg)
    assert out.shape == (qlen, B, H) and torch.equal(out, out2)
    # post-LN layer: rows are normalised before gamma/beta
    g, bt = w["layer_0/ff_ln/gamma"], w["layer_0/ff_ln/beta"]
    z = (out - bt) / g
    assert z.mean(-1).abs().max() < 1e-9 and (z.var(-1, unbiased=False) - 1).abs().max() < 1e-6


def test_gelu_tanh_and_layernorm_eps():
    x = torch.linspace(-4, 4, 101, dtype=D)
    assert torch.allclose(ox.gelu_tanh(x), torch.nn.functional.gelu(x, approximate="tanh"), atol=1e-14)
    y = torch.randn(3, 16, dtype=D)
    assert torch.allclose(ox.layer_norm(y, torch.ones(16, dtype=D), torch.zeros(16, dtype=D)),
                          torch.nn.functional.layer_norm(y, (16,), eps=1e-14), atol=1e-12)


def test_fully_masked_row_is_uniform():
    # the first position of a factorization order sees nothing in the query stream when there is no memory
    qlen, B, H, N, w, xs, mem, seg, _ = _tiny(0, 1)
    mask = torch.ones(qlen, qlen, B, dtype=D)
    d = H // N
    q = torch.randn(qlen, B, N, d, dtype=D)
    k = torch.randn(qlen, B, N, d, dtype=D)
    v = torch.randn(qlen, B, N, d, dtype=D)
    kr = torch.randn(2 * qlen, B, N, d, dtype=D)
    z = torch.zeros(N, d, dtype=D)
    vec = ox.rel_attn_core(q, k, v, kr, torch.zeros(2, N, d, dtype=D), ox.seg_mat_from_ids(seg), z, z, z, mask, 1.0)
    assert torch.allclose(vec, v.mean(0, keepdim=True).expand_as(vec), atol=1e-12)
