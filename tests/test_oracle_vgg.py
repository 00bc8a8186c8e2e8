"""Pins the VGG oracle: brute-force conv / pool, padding, ReLU-at-zero, parameter counts."""
import numpy as np
import torch

from dapple_amd import synthetic
from oracle import vgg as ov

D = torch.float64


def test_conv_same_padding_vs_brute_force():
    r = np.random.Generator(np.random.PCG64(1))
    x = r.standard_normal((2, 5, 4, 3))
    k = r.standard_normal((3, 3, 3, 2))
    b = r.standard_normal(2)
    want = np.zeros((2, 5, 4, 2))
    for n in range(2):
        for y in range(5):
            for xx in range(4):
                for co in range(2):
                    s = b[co]
                    for ky in range(3):
                        for kx in range(3):
                            yy, xc = y + ky - 1, xx + kx - 1
                            if 0 <= yy < 5 and 0 <= xc < 4:
                                for c in range(3):
                                    s += x[n, yy, xc, c] * k[ky, kx, c, co]
                    want[n, y, xx, co] = max(s, 0.0)
    got = ov.conv3x3_relu(torch.tensor(x), torch.tensor(k), torch.tensor(b))
    assert np.allclose(got.numpy(), want, atol=1e-12)


def test_max_pool_vs_brute_force_and_first_max_gradient():
    x = torch.randn(2, 6, 4, 3, dtype=D)
    got = ov.max_pool_2x2(x)
    for n in range(2):
        for y in range(3):
            for xx in range(2):
                for c in range(3):
                    assert got[n, y, xx, c] == x[n, 2 * y:2 * y + 2, 2 * xx:2 * xx + 2, c].max()
    xr = x.clone().requires_grad_(True)
    (g,) = torch.autograd.grad(ov.max_pool_2x2(xr).sum(), xr)
    assert g.sum().item() == 2 * 3 * 2 * 3 and set(g.unique().tolist()) == {0.0, 1.0}


def test_relu_gradient_is_zero_at_zero():
    x = torch.zeros(1, 2, 2, 1, dtype=D, requires_grad=True)
    k = torch.zeros(3, 3, 1, 1, dtype=D)
    b = torch.zeros(1, dtype=D, requires_grad=True)
    (gb,) = torch.autograd.grad(ov.conv3x3_relu(x, k, b).sum(), b)
    assert gb.item() == 0.0


def test_parameter_counts_match_reference_profile():
    # 16 convs = 20 024 384 parameters, the reference's 14-conv split 15 304 768
    def count(layers):
        return sum(v.size for v in synthetic.vgg_weights(0, synthetic.scale_layers(layers, 1)).values())
    assert count(synthetic.VGG19_CONV_STACK) == 20024384
    assert count(synthetic.VGG19_STAGE0_15_1) == 15304768
    assert ov.VGG19_CONV_STACK == synthetic.VGG19_CONV_STACK


def test_stage_vjp_finite_differences():
    layers = [("c1", 4), ("c2", 4), ("p1", None), ("c3", 8)]
    w = ov.to_torch(synthetic.vgg_weights(3, layers, perturb=True), requires_grad=True)
    x = torch.randn(1, 4, 4, 3, dtype=D)
    dy = torch.randn(1, 2, 2, 8, dtype=D)
    out, dx, dw = ov.stage_vjp(x, w, dy, layers, need_input_grad=True)
    assert out.shape == (1, 2, 2, 8)
    f = lambda xx, ww: (ov.stage_forward(xx, ww, layers) * dy).sum().item()
    eps = 1e-6
    for name in w:
        wd = {k: v.detach().clone() for k, v in w.items()}
        flat = wd[name].view(-1)
        i = flat.numel() // 3
        flat[i] += eps
        fp = f(x, wd)
        flat[i] -= 2 * eps
        fm = f(x, wd)
        assert abs((fp - fm) / (2 * eps) - dw[name].reshape(-1)[i].item()) < 1e-5, name


def test_forced_branches_reproduce_the_free_pass_and_follow_a_flipped_branch():
    """stage_vjp_forced_branches: (1) with the branches the oracle's own forward pass took it equals stage_vjp exactly;
    (2) with one ReLU mask entry and one pool pick flipped it equals finite differences of the function that takes those
    branches (scalar loops over the layers would say the same: the forced pass is multilinear, so central differences
    are exact up to rounding)."""
    r = np.random.Generator(np.random.PCG64(9))
    layers = [("c1", 4), ("p1", None), ("c2", 3)]
    x = torch.tensor(r.standard_normal((2, 4, 4, 2)))
    w = {"c1/kernel": torch.tensor(r.standard_normal((3, 3, 2, 4)) * 0.5), "c1/bias": torch.tensor(r.standard_normal(4) * 0.1),
         "c2/kernel": torch.tensor(r.standard_normal((3, 3, 4, 3)) * 0.5), "c2/bias": torch.tensor(r.standard_normal(3) * 0.1)}
    w = {k: v.requires_grad_(True) for k, v in w.items()}
    dy = torch.tensor(r.standard_normal((2, 2, 2, 3)))
    masks, picks = ov.branches_of(x, w, layers)
    out0, dx0, dw0 = ov.stage_vjp(x, w, dy, layers, need_input_grad=True)
    out1, dx1, dw1 = ov.stage_vjp_forced_branches(x, w, dy, layers, masks, picks, need_input_grad=True)
    assert torch.equal(out0, out1) and torch.allclose(dx0, dx1, atol=1e-14)
    for k in dw0:
        assert torch.allclose(dw0[k], dw1[k], atol=1e-14), k
    # flip one mask entry and one pick: the forced function changes, and its derivative follows
    masks["c1"][0, 1, 2, 3] = ~masks["c1"][0, 1, 2, 3]
    picks["p1"][1, 0, 1, 2] = (picks["p1"][1, 0, 1, 2] + 1) % 4
    _, _, dwf = ov.stage_vjp_forced_branches(x, w, dy, layers, masks, picks)

    def f(wd):
        out, _, _ = ov.stage_vjp_forced_branches(x, wd, dy, layers, masks, picks)
        return float((out * dy).sum())

    for name, idx in (("c1/kernel", (1, 2, 0, 3)), ("c2/kernel", (0, 1, 2, 1)), ("c1/bias", (3,)), ("c2/bias", (0,))):
        eps = 1e-5
        wp = {k: v.detach().clone().requires_grad_(True) for k, v in w.items()}
        wm = {k: v.detach().clone().requires_grad_(True) for k, v in w.items()}
        with torch.no_grad():
            wp[name][idx] += eps
            wm[name][idx] -= eps
        fd = (f(wp) - f(wm)) / (2 * eps)
        assert abs(fd - float(dwf[name][idx])) <= 1e-7 * max(1.0, abs(fd)), (name, fd, float(dwf[name][idx]))
    assert not torch.allclose(dwf["c1/kernel"], dw0["c1/kernel"])       # the flip is visible in the gradient


def _head_weights(r, features, fc, classes):
    return {"fc1/kernel": torch.tensor(r.standard_normal((features, fc)) * 0.3), "fc1/bias": torch.tensor(r.standard_normal(fc) * 0.1),
            "fc2/kernel": torch.tensor(r.standard_normal((fc, fc)) * 0.3), "fc2/bias": torch.tensor(r.standard_normal(fc) * 0.1),
            "predictions/kernel": torch.tensor(r.standard_normal((fc, classes)) * 0.3),
            "predictions/bias": torch.tensor(r.standard_normal(classes) * 0.1)}


def test_classification_block_vs_scalar_loops():
    r = np.random.Generator(np.random.PCG64(11))
    B, Fe, Fc, Cl = 3, 5, 4, 6
    hw = _head_weights(r, Fe, Fc, Cl)
    x = r.standard_normal((B, Fe))
    got = ov.head_forward(torch.tensor(x), hw).numpy()
    for b in range(B):
        h1 = [max(0.0, sum(x[b, i] * hw["fc1/kernel"][i, j].item() for i in range(Fe)) + hw["fc1/bias"][j].item()) for j in range(Fc)]
        h2 = [max(0.0, sum(h1[i] * hw["fc2/kernel"][i, j].item() for i in range(Fc)) + hw["fc2/bias"][j].item()) for j in range(Fc)]
        z = [sum(h2[i] * hw["predictions/kernel"][i, j].item() for i in range(Fc)) + hw["predictions/bias"][j].item() for j in range(Cl)]
        e = [np.exp(v - max(z)) for v in z]
        assert np.allclose(got[b], [v / sum(e) for v in e], atol=1e-12)


def test_losses_of_the_classification_block():
    r = np.random.Generator(np.random.PCG64(12))
    B, Cl = 4, 7
    z = torch.tensor(r.standard_normal((B, Cl)), requires_grad=True)
    p = torch.softmax(z, -1)
    labels = torch.tensor([3.0, 1.0, 6.0, 2.0])
    # the conventional loss is torch's cross_entropy on the logits
    want = torch.nn.functional.cross_entropy(z, labels.long())
    assert torch.allclose(ov.head_loss(p, labels, "sparse_ce"), want, atol=1e-12)
    # keras' function, used the right way round, is the one-hot cross entropy as well
    onehot = torch.nn.functional.one_hot(labels.long(), Cl).double()
    assert torch.allclose(ov.keras_categorical_crossentropy(onehot, p).mean(), want, atol=1e-6)    # (clipping at 1e-7)
    # as the reference calls it the label column is normalised to 1 and clipped: a constant, whatever the logits
    loss = ov.head_loss(p, labels, "as_written")
    assert abs(loss.item() - (-np.log(1.0 - 1e-7))) < 1e-15
    (g,) = torch.autograd.grad(loss, z)
    assert g.abs().max().item() < 1e-20 + 1e-7 * 1e-15          # constant upstream gradient dies in the softmax
    # a zero label is 0/0
    assert torch.isnan(ov.head_loss(p.detach(), torch.tensor([3.0, 0.0, 6.0, 2.0]), "as_written"))
