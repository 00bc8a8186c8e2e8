"""SQuAD-2 head of the last XLNet stage through the C ABI against the CPU oracle (autograd on the line-by-line
restatement of XLnetLoss.call), and a last-stage step: stage forward -> head -> stage backward."""
import numpy as np
import pytest
import torch

from dapple_amd import ops
from oracle import head as oh
from util import assert_close, dev

pytestmark = pytest.mark.gpu

NAMES = ("start_w", "start_b", "end_w0", "end_b0", "ln_gamma", "ln_beta", "end_w1", "end_b1", "ans_w0", "ans_b0", "ans_w1")


def make_case(seed, S, B, H, std):
    r = np.random.default_rng(seed)
    w = {n: r.standard_normal(ops.XLNET_HEAD_SHAPES[n](H)) * (std if n.endswith(("w", "w0", "w1")) else 0.1) for n in NAMES}
    w["ln_gamma"] = 1.0 + 0.1 * r.standard_normal(H)
    x = r.standard_normal((S, B, H))
    p_mask = (r.random((B, S)) < 0.3).astype(np.float64)
    p_mask[:, 0] = 0.0
    idx = lambda: r.integers(0, S, B).astype(np.int32)
    cls, sp, ep = idx(), idx(), idx()
    for b in range(B):                                       # labels sit on unmasked tokens, as in the data
        p_mask[b, sp[b]] = 0.0
        p_mask[b, ep[b]] = 0.0
    imp = (r.random(B) < 0.5).astype(np.float64)
    drop = (r.random((B, H)) >= 0.1).astype(np.float64) / 0.9
    return w, x, p_mask, cls, sp, ep, imp, drop


def oracle_run(w, x, p_mask, cls, sp, ep, imp, drop, x_rounded=None):
    wo = {n: torch.tensor(v, dtype=torch.float64).reshape(-1, 1).requires_grad_(True) if n in ("start_w", "end_w1", "ans_w1")
          else torch.tensor(v, dtype=torch.float64).requires_grad_(True) for n, v in w.items()}
    xo = (torch.tensor(x, dtype=torch.float64) if x_rounded is None else x_rounded.cpu().double()).requires_grad_(True)
    t = lambda a: torch.tensor(a)
    loss, sl, el, cl = oh.xlnet_squad_loss(xo, wo, t(cls), t(sp), t(ep), torch.tensor(imp, dtype=torch.float64),
                                           torch.tensor(p_mask, dtype=torch.float64),
                                           None if drop is None else torch.tensor(drop, dtype=torch.float64))
    grads = torch.autograd.grad(loss, [xo] + [wo[n] for n in NAMES])
    return loss, sl, el, cl, grads[0], {n: g.reshape(w[n].shape) for n, g in zip(NAMES, grads[1:])}


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("S,B,H,std,with_drop", [(16, 2, 64, 0.2, True), (37, 3, 72, 0.2, False), (512, 1, 1024, 0.02, True),
                                                 (128, 4, 256, 0.05, True)])
def test_xlnet_squad_head_matches_oracle(dtype, tol, S, B, H, std, with_drop):
    w, x, p_mask, cls, sp, ep, imp, drop = make_case(S * 7 + B + H, S, B, H, std)
    if B > 2:
        sp[-1] = S + 5                                       # tf.one_hot outside the range: zero feature, no start loss term
        cls[0] = -1
    if not with_drop:
        drop = None
    xd = dev(x, dtype)
    wd = {n: dev(v, torch.float32) for n, v in w.items()}
    gd = {n: torch.ones_like(v) for n, v in wd.items()}     # pre-filled: the head adds into the master gradients
    i32 = lambda a: torch.as_tensor(a).cuda()
    loss, sl, el, cl, dx = ops.xlnet_squad_head(xd, wd, i32(cls), i32(sp), i32(ep), dev(imp, torch.float32), dev(p_mask, torch.float32),
                                                None if drop is None else dev(drop, torch.float32), grads=gd, loss_scale=2.0)
    lo, slo, elo, clo, gx, gw = oracle_run(w, x, p_mask, cls, sp, ep, imp, drop, x_rounded=xd)
    assert_close(loss, 2.0 * lo.reshape(1), tol, "loss")
    assert_close(sl, slo, tol, "start logits")
    assert_close(el, elo, tol, "end logits")
    assert_close(cl, clo, tol, "cls logits")
    assert_close(dx, 2.0 * gx, tol, "dx")
    big = max(float(g.abs().max()) for g in gw.values())
    for n in NAMES:
        # the sum over the sequence of (softmax - one_hot) is zero, so the gradients of start_b, end_b1 and ln_beta
        # (= end_w1 times that sum) vanish identically: those are judged on the scale of the largest gradient
        assert_close(gd[n] - 1, 2.0 * gw[n], tol, "d " + n, floor=2.0 * big)


def test_forward_only_and_dx_only_agree_with_the_full_call():
    S, B, H = 24, 2, 64
    w, x, p_mask, cls, sp, ep, imp, drop = make_case(11, S, B, H, 0.2)
    xd = dev(x, torch.float32)
    wd = {n: dev(v, torch.float32) for n, v in w.items()}
    i32 = lambda a: torch.as_tensor(a).cuda()
    args = (xd, wd, i32(cls), i32(sp), i32(ep), dev(imp, torch.float32), dev(p_mask, torch.float32), dev(drop, torch.float32))
    gd = {n: torch.zeros_like(v) for n, v in wd.items()}
    full = ops.xlnet_squad_head(*args, grads=gd)
    fwd = ops.xlnet_squad_head(*args, need_dx=False)
    dxo = ops.xlnet_squad_head(*args)
    assert fwd[4] is None
    for a, b in zip(full[:4], fwd[:4]):                      # sums over the sequence go through atomics: equal to rounding
        assert_close(a, b.double().cpu(), 1e-6, "forward-only outputs")
    assert_close(full[4], dxo[4].double().cpu(), 1e-5, "dx without weight gradients")
    # a second call adds the same gradients again (accumulation over micro-batches)
    g1 = {n: v.clone() for n, v in gd.items()}
    ops.xlnet_squad_head(*args, grads=gd)
    big = max(float(v.abs().max()) for v in g1.values())
    for n in NAMES:                                          # start_b, end_b1, ln_beta are rounding noise around zero
        assert_close(gd[n], 2 * g1[n].double().cpu(), 1e-5, "accumulated d " + n, floor=1e3 * big if n in ("start_b", "end_b1", "ln_beta") else None)


def test_bad_arguments_are_rejected():
    S, B, H = 8, 1, 16
    w, x, p_mask, cls, sp, ep, imp, drop = make_case(3, S, B, H, 0.2)
    wd = {n: dev(v, torch.float32) for n, v in w.items()}
    i32 = lambda a: torch.as_tensor(a).cuda()
    with pytest.raises(ValueError):
        ops.xlnet_squad_head(dev(x, torch.float32), dict(wd, end_w0=wd["end_w0"][:H]), i32(cls), i32(sp), i32(ep), dev(imp, torch.float32),
                             dev(p_mask, torch.float32))
    with pytest.raises(ValueError):                          # hidden must be a multiple of 8
        x12 = dev(np.zeros((S, B, 12)), torch.float32)
        w12 = {n: torch.zeros(ops.XLNET_HEAD_SHAPES[n](12), device="cuda") for n in NAMES}
        ops.xlnet_squad_head(x12, w12, i32(cls), i32(sp), i32(ep), dev(imp, torch.float32), dev(p_mask, torch.float32))


def test_last_stage_step_with_the_head():
    # the last stage of a 2-stage XLNet (slice_xlnet.py:225-246): layers on the content stream, then XLnetLoss;
    # M micro-batches in the last stage's 1F1B order (K = 1: F0 B0 F1 B1), gradients accumulated over micro-batches
    from dapple_amd import runtime, synthetic
    from oracle import xlnet as ox
    L, H, N, F, B, Q, M = 2, 64, 4, 128, 2, 16, 2
    w_np = synthetic.xlnet_weights(41, L, H, N, F, stddev=0.1, perturb=True)
    xs_np = synthetic.xlnet_stream_inputs(42, M, Q, B, H, streams=1)
    r = np.random.Generator(np.random.PCG64(43))
    seg_ids = (r.random((Q, B)) > 0.6).astype(np.int64)
    im = (r.random((B, Q)) > 0.8).astype(np.int64)
    mask_t = ox.attn_mask_from_input_mask(torch.from_numpy(im), 0)
    hw, _, p_mask, _, _, _, _, _ = make_case(44, Q, B, H, 0.2)
    labels = [make_case(45 + j, Q, B, H, 0.2)[3:] for j in range(M)]

    st = runtime.xlnet_stage(L, H, N, F, B, Q, "fp32", stash_slots=1)
    st.bind(w_np)
    masks = dev(mask_t.numpy().astype(np.float32)[None])
    seg_mat = dev(ox.seg_mat_from_ids(torch.from_numpy(seg_ids), 0).numpy().astype(np.uint8))
    hwd = {n: dev(v, torch.float32) for n, v in hw.items()}
    hgd = {n: torch.zeros_like(v) for n, v in hwd.items()}
    i32 = lambda a: torch.as_tensor(a).cuda()
    losses, dxs = [], []
    for j in range(M):
        cls, sp, ep, imp, drop = labels[j]
        x = dev(np.stack(xs_np[j]), torch.float32)          # [1, Q, B, H]
        y = torch.empty_like(x)
        st.set_inputs(0, masks, seg_mat, None)
        st.forward(0, x, y)
        loss, _, _, _, dy = ops.xlnet_squad_head(y[0], hwd, i32(cls), i32(sp), i32(ep), dev(imp, torch.float32), dev(p_mask, torch.float32),
                                                 dev(drop, torch.float32), grads=hgd)
        dx = torch.empty_like(x)
        st.backward(0, dy.reshape(1, Q, B, H), dx)
        losses.append(loss)
        dxs.append(dx)
    st.sync()

    wt = ox.to_torch(w_np, torch.float64, requires_grad=True)
    hwo = {n: torch.tensor(v, dtype=torch.float64).reshape(-1, 1).requires_grad_(True) if n in ("start_w", "end_w1", "ans_w1")
           else torch.tensor(v, dtype=torch.float64).requires_grad_(True) for n, v in hw.items()}
    names = sorted(wt)
    acc = None
    for j in range(M):
        cls, sp, ep, imp, drop = labels[j]
        xo = torch.tensor(xs_np[j][0], dtype=torch.float64).requires_grad_(True)
        (yo,) = ox.stage_forward([xo], None, wt, list(range(L)), N, [mask_t.double()], torch.from_numpy(seg_ids))
        t = torch.tensor
        lo, _, _, _ = oh.xlnet_squad_loss(yo, hwo, t(cls), t(sp), t(ep), t(imp), t(p_mask), t(drop))
        params = [hwo[n] for n in NAMES] + [wt[n] for n in names]
        gs = torch.autograd.grad(lo, [xo] + params, allow_unused=True)
        assert_close(losses[j], lo.reshape(1), 1e-4, "loss mb%d" % j)
        assert_close(dxs[j][0], gs[0], 1e-4, "input grad mb%d" % j)
        gs = [torch.zeros_like(p) if g is None else g for g, p in zip(gs[1:], params)]
        acc = gs if acc is None else [a + g for a, g in zip(acc, gs)]
    big = max(float(g.abs().max()) for g in acc[:len(NAMES)])
    for n, g in zip(NAMES, acc):
        assert_close(hgd[n], g.reshape(hgd[n].shape), 1e-4, "head grad " + n, floor=big)
    for n, g in zip(names, acc[len(NAMES):]):
        if n not in st.grads:
            continue
        assert_close(st.grads[n], g.reshape(st.grads[n].shape), 1e-4, "stage grad " + n, floor=1e-3 * big if float(g.abs().max()) == 0 else None)
    st.close()
