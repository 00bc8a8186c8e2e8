"""Pins of oracle/amoeba.py (CPU): every operator against scalar loops over its published definition on small inputs, the
cell graph against a hand-written walk of amoeba_net_a's normal cell, and the reference's own cell specifications."""
import numpy as np
import torch

from dapple_amd import amoeba, synthetic
from oracle import amoeba as oa

D = torch.float64


def _rand(shape, seed):
    return torch.from_numpy(np.random.default_rng(seed).standard_normal(shape))


def test_depthwise_and_factorised_convolutions_against_loops():
    n, h, w, c, k = 2, 5, 4, 3, 3
    x, wt = _rand((n, h, w, c), 1), _rand((k, k, c), 2)
    ref = torch.zeros(n, h, w, c, dtype=D)
    for i in range(n):
        for y in range(h):
            for z in range(w):
                for ch in range(c):
                    s = 0.0
                    for a in range(k):
                        for b in range(k):
                            yy, zz = y + a - 1, z + b - 1
                            if 0 <= yy < h and 0 <= zz < w:
                                s += x[i, yy, zz, ch] * wt[a, b, ch]
                    ref[i, y, z, ch] = s
    assert torch.allclose(oa.depthwise_same(x, wt), ref, atol=1e-12)
    # 1 x 5 along the width, full convolution: w [1, 5, cin, cout]
    cin, cout, k = 3, 2, 5
    x, wt = _rand((n, h, w, cin), 3), _rand((1, k, cin, cout), 4)
    ref = torch.zeros(n, h, w, cout, dtype=D)
    for i in range(n):
        for y in range(h):
            for z in range(w):
                for t in range(k):
                    zz = z + t - k // 2
                    if 0 <= zz < w:
                        ref[i, y, z] += x[i, y, zz] @ wt[0, t]
    assert torch.allclose(oa.conv2d_same(x, wt), ref, atol=1e-12)
    wt = _rand((k, 1, cin, cout), 5)
    ref = torch.zeros(n, h, w, cout, dtype=D)
    for y in range(h):
        for t in range(k):
            yy = y + t - k // 2
            if 0 <= yy < h:
                ref[:, y] += x[:, yy] @ wt[t, 0]
    assert torch.allclose(oa.conv2d_same(x, wt), ref, atol=1e-12)


def test_pooling_same_padding_counts_only_taps_inside_the_image():
    x = _rand((1, 3, 4, 2), 6)
    for kind in ("avg", "max"):
        ref = torch.zeros_like(x)
        for y in range(3):
            for z in range(4):
                win = x[0, max(y - 1, 0):y + 2, max(z - 1, 0):z + 2].reshape(-1, 2)
                ref[0, y, z] = win.mean(0) if kind == "avg" else win.max(0).values
        assert torch.allclose(oa.pool3x3(x, kind), ref, atol=1e-12)
    ones = torch.ones(1, 5, 5, 1, dtype=D)
    assert torch.allclose(oa.pool3x3(ones, "avg"), ones)          # a constant image stays constant up to the border


def test_batch_norm_training_mode_and_moving_averages():
    x, g, b = _rand((4, 3, 3, 5), 7) * 3 + 2, _rand((5,), 8), _rand((5,), 9)
    y = oa.batch_norm_train(x, g, b)
    flat = x.reshape(-1, 5)
    for c in range(5):
        col = flat[:, c]
        m = col.sum() / col.numel()
        v = ((col - m) ** 2).sum() / col.numel()
        assert torch.allclose(y.reshape(-1, 5)[:, c], (col - m) / torch.sqrt(v + 1e-3) * g[c] + b[c], atol=1e-12)
    # with gamma = 1, beta = 0 the output has zero mean and variance var / (var + eps)
    y1 = oa.batch_norm_train(x, torch.ones(5, dtype=D), torch.zeros(5, dtype=D)).reshape(-1, 5)
    assert torch.allclose(y1.mean(0), torch.zeros(5, dtype=D), atol=1e-12)
    mm, mv = oa.moving_average_update(torch.zeros(5, dtype=D), torch.ones(5, dtype=D), x, 0.9)
    assert torch.allclose(mm, 0.1 * flat.mean(0)) and torch.allclose(mv, 0.9 + 0.1 * flat.var(0, unbiased=True))


def test_cell_specifications_are_the_references():
    # amoeba_net/model_specs.py:22-54; each cell has five combinations of two operations over seven hidden states
    for name, (ops_, idx, used) in synthetic.AMOEBA_NORMAL_CELLS.items():
        assert len(ops_) == 10 and len(idx) == 10 and len(used) == 7
        for it in range(5):
            assert max(idx[2 * it], idx[2 * it + 1]) < 2 + it       # a combination only reads states that exist
        assert used[6] == 0                                          # the last combination always reaches the output
    assert synthetic.AMOEBA_NORMAL_CELLS["amoeba_net_d"][0][3] == "1x7_7x1"


def test_cell_graph_of_amoeba_net_a_against_a_hand_written_walk():
    ops_, idx, used = synthetic.AMOEBA_NORMAL_CELLS["amoeba_net_a"]
    f, cin, cprev = 8, 12, 16
    shapes = amoeba.cell_variable_shapes("cell_0", cin, cprev, f, ops_, idx, used)
    p = {n: torch.from_numpy(v).double() for n, v in synthetic.amoeba_cell_weights(3, shapes).items()}
    net, prev = _rand((2, 6, 6, cin), 10), _rand((2, 6, 6, cprev), 11)
    out, (cut_prev, cut_net) = oa.cell_forward(net, prev, p, "cell_0", f, ops_, idx, used)
    bn = lambda t, s: oa.batch_norm_train(t, p["cell_0/%s/gamma" % s], p["cell_0/%s/beta" % s])

    def sep(t, side, it, k):
        for j in (1, 2):
            s = "cell_0/comb_iter_%d/%s/separable_%dx%d_%d" % (it, side, k, k, j)
            t = oa.depthwise_same(torch.relu(t), p[s + "/depthwise_weights"]) @ p[s + "/pointwise_weights"]
            t = bn(t, "comb_iter_%d/%s/bn_sep_%dx%d_%d" % (it, side, k, k, j))
        return t
    assert torch.equal(cut_prev, torch.relu(prev) @ p["cell_0/prev_1x1/weights"]) and torch.equal(cut_net, torch.relu(net) @ p["cell_0/1x1/weights"])
    h0, h1 = bn(cut_net, "beginning_bn"), bn(cut_prev, "prev_bn")
    h2 = oa.pool3x3(h0, "avg") + oa.pool3x3(h0, "max")
    h3 = sep(h1, "left", 1, 3) + h1
    h4 = h0 + oa.pool3x3(h1, "avg")
    h5 = sep(h0, "left", 3, 3) + sep(h2, "right", 3, 5)
    h6 = oa.pool3x3(h5, "avg") + sep(h0, "right", 4, 3)
    assert out.shape == (2, 6, 6, 4 * f)
    assert torch.allclose(out, torch.cat([h1, h3, h4, h6], -1), atol=1e-12)      # used = [1, 0, 1, 0, 0, 1, 0]


def test_cell_vjp_against_finite_differences():
    ops_, idx, used = synthetic.AMOEBA_NORMAL_CELLS["amoeba_net_d"]
    f, cin = 8, 8
    shapes = amoeba.cell_variable_shapes("cell_1", cin, cin, f, ops_, idx, used)
    p = {n: torch.from_numpy(v).double() for n, v in synthetic.amoeba_cell_weights(5, shapes).items()}
    net, prev, d_out = _rand((2, 4, 4, cin), 12), _rand((2, 4, 4, cin), 13), _rand((2, 4, 4, 4 * f), 14)
    out, d_net, d_prev, dw = oa.cell_vjp(net, prev, p, d_out, "cell_1", f, ops_, idx, used)
    loss = lambda n_, pr, pp: (oa.cell_forward(n_, pr, pp, "cell_1", f, ops_, idx, used)[0] * d_out).sum()
    e = 1e-6
    for pos in [(0, 1, 2, 3), (1, 3, 0, 5)]:
        for which, g in (("net", d_net), ("prev", d_prev)):
            a, b = net.clone(), prev.clone()
            t = a if which == "net" else b
            t[pos] += e
            up = loss(a, b, p)
            t[pos] -= 2 * e
            assert abs((up - loss(a, b, p)) / (2 * e) - g[pos]) < 1e-6 * max(1.0, abs(g[pos]))
    name = "cell_1/comb_iter_1/right/1x7/weights"
    q = dict(p)
    q[name] = p[name].clone()
    q[name][3, 1] += e
    up = loss(net, prev, q)
    q[name][3, 1] -= 2 * e
    assert abs((up - loss(net, prev, q)) / (2 * e) - dw[name][3, 1]) < 1e-6 * max(1.0, abs(dw[name][3, 1]))
