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


def test_regression_head_is_the_pairwise_mean_of_the_reference_graph():
    """bert.py:627-631 subtracts the [batch] label placeholder (bert_finetune.py:212) from the [batch, 1] prediction:
    the difference is [batch, batch].  Pinned by scalar loops over every pair, by the closed form
    mean_i (z_i - mean y)^2 + var(y), and by the case of one sample, where it is the plain squared error."""
    torch.manual_seed(5)
    B, S, H = 4, 3, 6
    x = torch.randn(B, S, H, dtype=torch.float64)
    wp, bp = torch.randn(H, H, dtype=torch.float64) * 0.5, torch.randn(H, dtype=torch.float64) * 0.1
    wf = (torch.randn(H, 1, dtype=torch.float64) * 0.5).requires_grad_(True)
    bf = torch.full((1,), 1e-4, dtype=torch.float64)
    y = torch.randn(B, dtype=torch.float64)
    loss, pred, pooled = oh.regression_loss(x, wp, bp, wf, bf, y, l2_scale=1e-3)
    assert tuple(pred.shape) == (B, 1)
    z = []
    for b in range(B):
        pz = [math.tanh(sum(x[b, 0, i].item() * wp[i, j].item() for i in range(H)) + bp[j].item()) for j in range(H)]
        z.append(sum(pz[j] * wf[j, 0].item() for j in range(H)) + bf[0].item())
        assert abs(z[b] - pred[b, 0].item()) < 1e-12
    reg = 1e-3 * 0.5 * float((wf.detach() ** 2).sum())
    brute = sum((z[i] - y[j].item()) ** 2 for i in range(B) for j in range(B)) / (B * B)
    assert abs(loss.item() - (brute + reg)) < 1e-12
    ym = float(y.mean())
    closed = sum((zi - ym) ** 2 for zi in z) / B + float(((y - ym) ** 2).mean())
    assert abs(loss.item() - (closed + reg)) < 1e-12
    # d loss / d prediction_i = 2 (z_i - mean y) / B
    (g,) = torch.autograd.grad(loss, pred, retain_graph=True)
    assert torch.allclose(g[:, 0], torch.tensor([2 * (zi - ym) / B for zi in z], dtype=torch.float64), atol=1e-12)
    # one sample: the ordinary squared error
    l1, p1, _ = oh.regression_loss(x[:1], wp, bp, wf, bf, y[:1], l2_scale=0.0)
    assert abs(l1.item() - (p1[0, 0].item() - y[0].item()) ** 2) < 1e-12


def _xlnet_head_case(seed, S, B, H, std=0.3):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    w = dict(start_w=r(H, 1) * std, start_b=r(1) * 0.1, end_w0=r(2 * H, H) * std, end_b0=r(H) * 0.1,
             ln_gamma=1 + 0.1 * r(H), ln_beta=0.1 * r(H), end_w1=r(H, 1) * std, end_b1=r(1) * 0.1,
             ans_w0=r(2 * H, H) * std, ans_b0=r(H) * 0.1, ans_w1=r(H, 1) * std)
    out = r(S, B, H)
    p_mask = (torch.rand(B, S, generator=g) < 0.3).double()
    p_mask[:, 0] = 0.0
    return out, w, p_mask


def test_xlnet_squad_loss_matches_library_routines():
    S, B, H = 7, 3, 6
    out, w, p_mask = _xlnet_head_case(5, S, B, H)
    cls = torch.tensor([6, 0, 3]); sp = torch.tensor([0, 2, 5]); ep = torch.tensor([1, 4, 6])
    imp = torch.tensor([0.0, 1.0, 0.0], dtype=torch.float64)
    drop = torch.tensor([[0.0, 1 / 0.9] * (H // 2)] * B, dtype=torch.float64)
    loss, sl, el, cl = oh.xlnet_squad_loss(out, w, cls, sp, ep, imp, p_mask, drop)
    F = torch.nn.functional
    # start branch: a Linear over the feature axis, transposed to [batch, seq]
    assert torch.allclose(sl, (out.permute(1, 0, 2) @ w["start_w"]).squeeze(-1) + w["start_b"], atol=1e-12)
    slm = torch.where(p_mask > 0, torch.full_like(sl, -1e30), sl)
    start_loss = F.cross_entropy(slm, sp)
    # end branch from library pieces: the one-hot einsum is a row pick; F.layer_norm with eps 1e-14
    picked = torch.stack([out[sp[b], b] for b in range(B)])
    cat = torch.cat([out, picked.unsqueeze(0).expand(S, B, H)], -1)
    e = F.layer_norm(torch.tanh(cat @ w["end_w0"] + w["end_b0"]), (H,), w["ln_gamma"], w["ln_beta"], eps=1e-14)
    el_ref = (e @ w["end_w1"]).squeeze(-1).t() + w["end_b1"]
    assert torch.allclose(el, el_ref, atol=1e-10)
    end_loss = F.cross_entropy(torch.where(p_mask > 0, torch.full_like(el, -1e30), el), ep)
    # answerability branch
    sf = (torch.softmax(slm, -1).t().unsqueeze(-1) * out).sum(0)
    cf = torch.stack([out[cls[b], b] for b in range(B)])
    a = torch.tanh(torch.cat([sf, cf], -1) @ w["ans_w0"] + w["ans_b0"]) * drop
    cl_ref = (a @ w["ans_w1"]).squeeze(-1)
    assert torch.allclose(cl, cl_ref, atol=1e-10)
    reg = F.binary_cross_entropy_with_logits(cl_ref, imp)
    assert abs(loss.item() - (0.5 * (start_loss + end_loss) + 0.5 * reg).item()) < 1e-10


def test_xlnet_squad_loss_brute_force_and_edge_cases():
    S, B, H = 4, 2, 2
    out, w, p_mask = _xlnet_head_case(6, S, B, H)
    p_mask[1, 2] = 1.0
    cls = torch.tensor([3, 0]); sp = torch.tensor([1, 0]); ep = torch.tensor([3, 1])
    imp = torch.tensor([1.0, 0.0], dtype=torch.float64)
    loss, sl, el, cl = oh.xlnet_squad_loss(out, w, cls, sp, ep, imp, p_mask)
    f = lambda t: t.tolist()
    o, pm = f(out), f(p_mask)
    sw, sb = [v[0] for v in f(w["start_w"])], w["start_b"].item()
    tot = 0.0
    for b in range(B):
        lg = [sum(o[l][b][h] * sw[h] for h in range(H)) + sb for l in range(S)]
        assert all(abs(lg[l] - sl[b, l].item()) < 1e-12 for l in range(S))
        lm = [lg[l] * (1 - pm[b][l]) - 1e30 * pm[b][l] for l in range(S)]
        mx = max(lm)
        z = sum(math.exp(v - mx) for v in lm)
        ps = [math.exp(v - mx) / z for v in lm]
        tot += -0.5 * (lm[sp[b]] - mx - math.log(z)) / B
        # end logits: concat(output[l, b], output[start, b]) -> dense tanh -> layer norm -> dense
        W0, b0 = f(w["end_w0"]), f(w["end_b0"])
        em = []
        for l in range(S):
            cat = o[l][b] + o[sp[b]][b]
            t = [math.tanh(sum(cat[k] * W0[k][j] for k in range(2 * H)) + b0[j]) for j in range(H)]
            mu = sum(t) / H
            var = sum((v - mu) ** 2 for v in t) / H
            n = [(t[j] - mu) / math.sqrt(var + 1e-14) * w["ln_gamma"][j].item() + w["ln_beta"][j].item() for j in range(H)]
            e = sum(n[j] * w["end_w1"][j, 0].item() for j in range(H)) + w["end_b1"].item()
            assert abs(e - el[b, l].item()) < 1e-9
            em.append(e * (1 - pm[b][l]) - 1e30 * pm[b][l])
        mx = max(em)
        tot += -0.5 * (em[ep[b]] - mx - math.log(sum(math.exp(v - mx) for v in em))) / B
        # answerability
        sfeat = [sum(ps[l] * o[l][b][h] for l in range(S)) for h in range(H)]
        cat = sfeat + o[cls[b]][b]
        W1, b1 = f(w["ans_w0"]), f(w["ans_b0"])
        a = [math.tanh(sum(cat[k] * W1[k][j] for k in range(2 * H)) + b1[j]) for j in range(H)]
        x = sum(a[j] * w["ans_w1"][j, 0].item() for j in range(H))
        assert abs(x - cl[b].item()) < 1e-10
        tot += 0.5 * (max(x, 0) - x * imp[b].item() + math.log(1 + math.exp(-abs(x)))) / B
    assert abs(loss.item() - tot) < 1e-10
    # a masked position gets probability zero; positions outside [0, seq) give no loss term and a zero start feature
    assert torch.softmax(sl * (1 - p_mask) - 1e30 * p_mask, -1)[1, 2].item() == 0.0
    l2, _, el2, _ = oh.xlnet_squad_loss(out, w, cls, torch.tensor([1, 9]), ep, imp, p_mask)
    zero_feat = torch.cat([out[:, 1], torch.zeros(S, H, dtype=torch.float64)], -1)
    e = torch.tanh(zero_feat @ w["end_w0"] + w["end_b0"])
    e = torch.nn.functional.layer_norm(e, (H,), w["ln_gamma"], w["ln_beta"], eps=1e-14)
    assert torch.allclose(el2[1], (e @ w["end_w1"]).squeeze(-1) + w["end_b1"], atol=1e-10)
