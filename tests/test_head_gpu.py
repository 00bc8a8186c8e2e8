"""SQuAD head through the C ABI against the CPU oracle, and a last-stage step: stage forward -> head ->
stage backward with the head's input gradient."""
import numpy as np
import pytest
import torch

from dapple_amd import ops, runtime, synthetic
from oracle import bert as ob
from oracle import head as oh
from util import assert_close, dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("B,S,H", [(2, 16, 64), (3, 384, 1024), (1, 5, 8)])
def test_squad_head_matches_oracle(dtype, tol, B, S, H):
    r = np.random.default_rng(B * S + H)
    x = dev(r.standard_normal((B * S, H)), dtype)
    w = dev(r.standard_normal((2, H)) * 0.1, torch.float32)
    b = dev(r.standard_normal(2) * 0.1, torch.float32)
    sp_np = r.integers(0, S, B).astype(np.int32)
    ep_np = r.integers(0, S, B).astype(np.int32)
    if B > 1:
        ep_np[-1] = S + 3                                   # tf.one_hot of an out-of-range index: no loss term
    sp, ep = torch.as_tensor(sp_np).cuda(), torch.as_tensor(ep_np).cuda()
    dw = torch.ones(2, H, device="cuda")                    # pre-filled: the head adds into the master gradients
    db = torch.ones(2, device="cuda")
    loss, sl, el, dx = ops.squad_head(x, B, S, w, b, sp, ep, dw, db)
    xo = x.cpu().double().reshape(B, S, H).requires_grad_(True)
    wo = w.cpu().double().requires_grad_(True)
    bo = b.cpu().double().requires_grad_(True)
    lo, slo, elo = oh.squad_loss(xo, wo, bo, torch.as_tensor(sp_np), torch.as_tensor(ep_np))
    gx, gw, gb = torch.autograd.grad(lo, [xo, wo, bo])
    assert_close(loss, lo.reshape(1), tol, "loss")
    assert_close(sl, slo, tol, "start logits")
    assert_close(el, elo, tol, "end logits")
    assert_close(dx, gx.reshape(B * S, H), tol, "dx")
    assert_close(dw - 1, gw, tol, "d output_weights")
    # sum over the sequence of (softmax - one_hot) is zero: the bias gradient vanishes identically, judge it on the
    # scale of the weight gradient
    assert_close(db - 1, gb, tol, "d output_bias", floor=float(gw.abs().max()))


def test_last_stage_step_with_the_head():
    # stage 1 of a 2-stage BERT: layers, then the SQuAD loss; M micro-batches under the 1F1B order for the last
    # stage (K = 1): F0 B0 F1 B1 ..., gradients accumulated over micro-batches
    L, H, N, F, B, S, M = 2, 64, 4, 128, 2, 16, 3
    w = synthetic.bert_weights(31, L, H, F)
    r = np.random.default_rng(32)
    hw_np, hb_np = r.standard_normal((2, H)) * 0.05, r.standard_normal(2) * 0.05
    xs_np = synthetic.bert_activation_inputs(33, M, B, S, H)
    sp_np = r.integers(0, S, (M, B)).astype(np.int32)
    ep_np = r.integers(0, S, (M, B)).astype(np.int32)
    st = runtime.bert_stage(L, H, N, F, B, S, "fp32", stash_slots=1)
    st.bind(w)
    hw, hb = dev(hw_np, torch.float32), dev(hb_np, torch.float32)
    dhw, dhb = torch.zeros_like(hw), torch.zeros_like(hb)
    losses, dxs = [], []
    for j in range(M):
        x = torch.as_tensor(xs_np[j]).cuda()
        y = torch.empty(B * S, H, device="cuda")
        st.forward(0, x, y)
        loss, _, _, dy = ops.squad_head(y, B, S, hw, hb, torch.as_tensor(sp_np[j]).cuda(), torch.as_tensor(ep_np[j]).cuda(), dhw, dhb)
        dx = torch.empty_like(x)
        st.backward(0, dy, dx)
        losses.append(loss)
        dxs.append(dx)
    st.sync()
    wt = ob.to_torch(w, torch.float64, requires_grad=True)
    hwo = torch.as_tensor(hw_np).requires_grad_(True)
    hbo = torch.as_tensor(hb_np).requires_grad_(True)
    names = list(wt)
    acc = None
    for j in range(M):
        xo = torch.as_tensor(xs_np[j]).double().requires_grad_(True)
        yo = ob.stage_forward(xo, wt, list(range(L)), B, S, N)
        lo, _, _ = oh.squad_loss(yo.reshape(B, S, H), hwo, hbo, torch.as_tensor(sp_np[j]), torch.as_tensor(ep_np[j]))
        gs = torch.autograd.grad(lo, [xo, hwo, hbo] + [wt[n] for n in names], allow_unused=True)
        assert_close(losses[j], lo.reshape(1), 1e-4, "loss mb%d" % j)
        assert_close(dxs[j], gs[0], 1e-4, "input grad mb%d" % j)
        gs = [torch.zeros_like(t) if g is None else g for g, t in zip(gs[1:], [hwo, hbo] + [wt[n] for n in names])]
        acc = gs if acc is None else [a + g for a, g in zip(acc, gs)]
    assert_close(dhw, acc[0], 1e-4, "d output_weights")
    assert_close(dhb, acc[1], 1e-4, "d output_bias", floor=float(acc[0].abs().max()))
    for n, g in zip(names, acc[2:]):
        floor = None
        if n.endswith("/key/bias"):
            floor = float(acc[2 + names.index(n.replace("/key/", "/query/"))].abs().max())
        if n.endswith("layer_%d/output/LayerNorm/beta" % (L - 1)):
            # d beta = column sums of the head's dx = w0 * sum(dlogits0) + w1 * sum(dlogits1) = 0 identically
            floor = float(acc[2 + names.index(n.replace("/beta", "/gamma"))].abs().max())
        assert_close(st.grads[n], g.reshape(st.grads[n].shape), 1e-4, "grad " + n, floor=floor)
    st.close()


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("B,S,H,C", [(2, 16, 64, 2), (3, 128, 1024, 2), (1, 4, 8, 5)])
def test_classifier_head_matches_oracle(dtype, tol, B, S, H, C):
    r = np.random.default_rng(B * S + H + C)
    x = dev(r.standard_normal((B * S, H)), dtype)
    wp = dev(r.standard_normal((H, H)) / np.sqrt(H), torch.float32)
    bp = dev(r.standard_normal(H) * 0.1, torch.float32)
    wf = dev(r.standard_normal((H, C)) * 0.3, torch.float32)
    bf = dev(np.full(C, 1e-4), torch.float32)                  # biases_initializer=constant(1e-04), bert.py:650
    y_np = r.integers(0, C, B).astype(np.int32)
    y = torch.as_tensor(y_np).cuda()
    grads = [torch.ones_like(t) for t in (wp, bp, wf, bf)]      # pre-filled: the head adds into the master gradients
    loss, logits, pooled, dx = ops.classifier_head(x, B, S, wp, bp, wf, bf, y, grads)
    xo = x.cpu().double().reshape(B, S, H).requires_grad_(True)
    ws = [t.cpu().double().requires_grad_(True) for t in (wp, bp, wf, bf)]
    lo, lgo, po = oh.classification_loss(xo, ws[0], ws[1], ws[2], ws[3], torch.as_tensor(y_np))
    gx, *gw = torch.autograd.grad(lo, [xo] + ws)
    assert_close(loss, lo.reshape(1), tol, "loss")
    assert_close(logits, lgo, tol, "logits")
    assert_close(pooled, po, tol, "pooled")
    assert_close(dx, gx.reshape(B * S, H), tol, "dx")
    assert float(dx.reshape(B, S, H)[:, 1:].abs().max() if S > 1 else 0.0) == 0.0   # only the first token has a gradient
    for g, ref, name in zip(grads, gw, ("pooler kernel", "pooler bias", "FC weights", "FC biases")):
        assert_close(g - 1, ref, tol, "d " + name, floor=float(gw[2].abs().max()) if name == "FC biases" else None)
    # loss_scale scales loss and gradients; no gradient buffers: forward only
    loss2, _, _, dx2 = ops.classifier_head(x, B, S, wp, bp, wf, bf, y, None, loss_scale=4.0)
    assert_close(loss2, 4 * lo.reshape(1), tol, "scaled loss")
    assert_close(dx2, 4 * gx.reshape(B * S, H), tol, "scaled dx")
    with pytest.raises(ValueError):
        ops.classifier_head(x, B, S, wp, bp, wf, bf, y.long())


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("B,S,H", [(2, 16, 64), (6, 128, 1024), (1, 4, 8)])
def test_regression_head_matches_oracle(dtype, tol, B, S, H):
    r = np.random.default_rng(B * S + H)
    x = dev(r.standard_normal((B * S, H)), dtype)
    wp = dev(r.standard_normal((H, H)) / np.sqrt(H), torch.float32)
    bp = dev(r.standard_normal(H) * 0.1, torch.float32)
    wf = dev(r.standard_normal((H, 1)) * 0.3, torch.float32)
    bf = dev(np.full(1, 1e-4), torch.float32)
    y_np = r.standard_normal(B).astype(np.float32)
    y = torch.as_tensor(y_np).cuda()
    grads = [torch.ones_like(t) for t in (wp, bp, wf, bf)]
    loss, pred, pooled, dx = ops.regression_head(x, B, S, wp, bp, wf, bf, y, grads)
    xo = x.cpu().double().reshape(B, S, H).requires_grad_(True)
    ws = [t.cpu().double().requires_grad_(True) for t in (wp, bp, wf, bf)]
    lo, po, zo = oh.regression_loss(xo, ws[0], ws[1], ws[2], ws[3], torch.as_tensor(y_np).double())
    gx, *gw = torch.autograd.grad(lo, [xo] + ws)
    assert_close(loss, lo.reshape(1), tol, "loss")
    assert_close(pred, po, tol, "prediction")
    assert_close(pooled, zo, tol, "pooled")
    assert_close(dx, gx.reshape(B * S, H), tol, "dx")
    for g, ref, name in zip(grads, gw, ("pooler kernel", "pooler bias", "FC weights", "FC biases")):
        assert_close(g - 1, ref, tol, "d " + name, floor=float(gw[2].abs().max()) if name == "FC biases" else None)
    loss2, _, _, dx2 = ops.regression_head(x, B, S, wp, bp, wf, bf, y, None, loss_scale=0.5)
    assert_close(loss2, 0.5 * lo.reshape(1), tol, "scaled loss")
    assert_close(dx2, 0.5 * gx.reshape(B * S, H), tol, "scaled dx")
    with pytest.raises(ValueError):
        ops.regression_head(x, B, S, wp, bp, wf, bf, y.double())
