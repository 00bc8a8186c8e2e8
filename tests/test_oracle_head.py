"""Pins of oracle/head.py (CPU)."""
import math

import torch

from oracle import head as oh


def test_matches_library_cross_entropy_and_brute_force():
    torch.manual_seed(0)
    B, S, H = 3, 5, 4
    x = torch.randn(B, S, H, dtype=torch.float64)
    w = torch.randn(2, H, dtype=torch.float64)
    b = torch.randn(2, dtype=torch.float64)
    sp = torch.tensor([0, 4, 2], dtype=torch.int32)
    ep = torch.tensor([1, 1, 3], dtype=torch.int32)
    loss, sl, el = oh.squad_loss(x, w, b, sp, ep)
    # library routine
    ref = (torch.nn.functional.cross_entropy(sl, sp.long()) + torch.nn.functional.cross_entropy(el, ep.long())) / 2
    assert abs(loss.item() - ref.item()) < 1e-12
    # brute force, including which weight row feeds which logit
    tot = 0.0
    for bb in range(B):
        for c, pos in ((0, sp), (1, ep)):
            lg = [sum(x[bb, s, h].item() * w[c, h].item() for h in range(H)) + b[c].item() for s in range(S)]
            lse = math.log(sum(math.exp(v) for v in lg))
            tot += -(lg[pos[bb].item()] - lse)
    assert abs(loss.item() - tot / (2 * B)) < 1e-12
    assert torch.allclose(sl[1], x[1] @ w[0] + b[0])


def test_out_of_range_position_gives_no_loss_term():
    torch.manual_seed(1)
    x = torch.randn(2, 4, 3, dtype=torch.float64)
    w = torch.randn(2, 3, dtype=torch.float64)
    b = torch.zeros(2, dtype=torch.float64)
    full, _, _ = oh.squad_loss(x, w, b, torch.tensor([1, 2]), torch.tensor([0, 3]))
    part, sl, _ = oh.squad_loss(x, w, b, torch.tensor([1, 9]), torch.tensor([0, 3]))
    missing = -torch.log_softmax(sl[1], -1)[2] / (2 * 2)
    assert abs((full - part).item() - missing.item()) < 1e-12


def test_classification_head_matches_library_and_brute_force():
    torch.manual_seed(2)
    B, S, H, C = 3, 4, 5, 2
    x = torch.randn(B, S, H, dtype=torch.float64)
    wp, bp = torch.randn(H, H, dtype=torch.float64) * 0.5, torch.randn(H, dtype=torch.float64) * 0.1
    wf = (torch.randn(H, C, dtype=torch.float64) * 0.5).requires_grad_(True)
    bf = torch.full((C,), 1e-4, dtype=torch.float64)
    y = torch.tensor([1, 0, 1])
    loss, logits, pooled = oh.classification_loss(x, wp, bp, wf, bf, y, l2_scale=1e-3)
    # library routines: Linear + tanh on the FIRST token, mean cross entropy; the regulariser by its closed form
    lin = torch.nn.Linear(H, H).double()
    with torch.no_grad():
        lin.weight.copy_(wp.t()); lin.bias.copy_(bp)
    assert torch.allclose(pooled, torch.tanh(lin(x[:, 0])), atol=1e-12)
    ce = torch.nn.functional.cross_entropy(pooled @ wf + bf, y)
    assert abs(loss.item() - (ce.item() + 1e-3 * 0.5 * float((wf.detach() ** 2).sum()))) < 1e-12
    # the gradient of the regulariser alone is scale * w (tf.nn.l2_loss = sum(w^2) / 2)
    (g_all,) = torch.autograd.grad(loss, wf, retain_graph=True)
    (g_ce,) = torch.autograd.grad(ce, wf)
    assert torch.allclose(g_all - g_ce, 1e-3 * wf.detach(), atol=1e-12)
    # brute force on one sample
    b = 2
    z = [math.tanh(sum(x[b, 0, i].item() * wp[i, j].item() for i in range(H)) + bp[j].item()) for j in range(H)]
    lg = [sum(z[j] * wf[j, c].item() for j in range(H)) + bf[c].item() for c in range(C)]
    assert abs(lg[0] - logits[b, 0].item()) < 1e-12 and abs(lg[1] - logits[b, 1].item()) < 1e-12
    # tokens other than the first do not enter
    x2 = x.clone(); x2[:, 1:] += 1.0
    assert abs(oh.classification_loss(x2, wp, bp, wf, bf, y)[0].item() - loss.item()) < 1e-12
