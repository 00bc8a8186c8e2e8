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
