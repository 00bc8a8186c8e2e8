"""The decoder cells of GNMT's second pipeline device through the C ABI against the fp64 CPU oracle (fp32: 1e-4)."""
import numpy as np
import pytest
import torch

from dapple_amd import runtime, synthetic
from oracle import gnmt as og
from util import assert_close, dev

pytestmark = pytest.mark.gpu
TOL = 1e-4


def run_case(L, U, B, T, M, K=1, first_layer=1, seed=0, init=0.3, attention="steps", overlap=False):
    w_np = synthetic.gnmt_decoder_weights(synthetic.SEED_WEIGHT + seed, first_layer, L, U, init_weight=init, perturb=True)
    r = np.random.Generator(np.random.PCG64(500 + seed))
    xs_np = [r.standard_normal((T, B, U)).astype(np.float32) for _ in range(M)]
    dys_np = synthetic.upstream_grads(synthetic.SEED_GRAD + seed, M, (T, B, U))
    if attention == "steps":
        att_np = [r.standard_normal((T, B, U)).astype(np.float32) for _ in range(M)]
    elif attention == "constant":     # one vector for all steps, as a variable read inside the loop gives
        att_np = [np.broadcast_to(r.standard_normal((1, B, U)).astype(np.float32), (T, B, U)).copy() for _ in range(M)]
    else:
        att_np = [None] * M
    stage = runtime.gnmt_decoder_stage(L, U, B, T, stash_slots=K, first_layer=first_layer)
    assert stage.weight_names == [s + sfx for s, _ in og.decoder_cell_names(first_layer, L) for sfx in ("/kernel", "/bias")]
    stage.bind(w_np)
    if overlap:
        stage.enable_overlap()
    xs, dys = [dev(x) for x in xs_np], [dev(d) for d in dys_np]
    atts = [None if a is None else dev(a) for a in att_np]
    outs = [torch.empty(T, B, U, device="cuda") for _ in range(M)]
    dxs = [torch.empty(T, B, U, device="cuda") for _ in range(M)]
    runtime.StageRuntime(stage, 0, K, M).step(xs, dys, outs, dxs, before_forward=lambda slot, j: stage.set_attention(slot, atts[j]))
    stage.sync()
    w_t = og.to_torch(w_np, torch.float64, requires_grad=True)
    names = sorted(w_t)
    acc = None
    for j in range(M):
        xo = torch.tensor(xs_np[j], dtype=torch.float64, requires_grad=True)
        ao = None if att_np[j] is None else torch.tensor(att_np[j], dtype=torch.float64)
        out = og.decoder_part2_forward(xo, ao, w_t, first_layer, L)
        gs = torch.autograd.grad(out, [xo] + [w_t[n] for n in names], grad_outputs=torch.tensor(dys_np[j], dtype=torch.float64))
        assert_close(outs[j], out.detach(), TOL, "output mb%d" % j)
        assert_close(dxs[j], gs[0], TOL, "input grad mb%d" % j)
        acc = list(gs[1:]) if acc is None else [a + g for a, g in zip(acc, gs[1:])]
    for n, g in zip(names, acc):
        got = stage.grads[n]
        if attention is None and n.endswith("/kernel"):
            assert float(got[U:2 * U].abs().max()) == 0.0          # zero attention: those rows get no gradient, exactly
        assert_close(got, g.reshape(got.shape), TOL, "accumulated grad " + n)
    stage.close()


def test_three_cells_with_per_step_attention():
    run_case(L=3, U=32, B=4, T=6, M=3, K=2)


def test_zero_attention_is_the_default():
    run_case(L=2, U=16, B=4, T=5, M=2, attention=None, seed=1)


def test_constant_attention_single_step_and_single_cell():
    run_case(L=1, U=16, B=8, T=1, M=2, attention="constant", seed=2)
    run_case(L=1, U=16, B=4, T=4, M=1, first_layer=2, attention="constant", seed=3)


def test_overlapped_streams():
    run_case(L=3, U=32, B=4, T=5, M=4, K=2, seed=4, overlap=True)


def test_reference_cell_shape():
    # units 1024, batch 64, 50 steps (BASELINE configs[2]'s cell shape): cell 1 (no residual) and cell 2 (residual)
    run_case(L=2, U=1024, B=64, T=50, M=1, seed=5, init=0.05)


def test_wrong_side_input_calls_are_rejected():
    dec = runtime.gnmt_decoder_stage(1, 16, 4, 3, stash_slots=1)
    with pytest.raises(ValueError):
        dec.set_lengths(0, torch.zeros(4, dtype=torch.int32, device="cuda"))
    with pytest.raises(ValueError):
        dec.set_attention(0, torch.zeros(3, 4, 8, device="cuda"))
    dec.close()
    enc = runtime.gnmt_stage(2, 16, 10, 4, 3, stash_slots=1)
    with pytest.raises(ValueError):
        enc.set_attention(0, torch.zeros(3, 4, 16, device="cuda"))
    enc.close()


@pytest.mark.parametrize("T,B,U,V,lens", [(5, 4, 16, 24, [5, 3, 0, 1]), (7, 3, 32, 100, [7, 7, 2]), (50, 64, 1024, 32000, None)])
def test_projection_and_loss_match_oracle(T, B, U, V, lens):
    from dapple_amd import ops
    r = np.random.Generator(np.random.PCG64(T * B + V))
    x_np = r.standard_normal((T, B, U)).astype(np.float32) * 0.5
    k_np = r.uniform(-0.1, 0.1, (U, V)).astype(np.float32)
    tgt_np = r.integers(0, V, (B, T)).astype(np.int32)
    lens_np = np.asarray(lens if lens is not None else r.integers(1, T + 1, B), dtype=np.int32)
    x, k = dev(x_np), dev(k_np)
    dk = torch.ones_like(k)                                    # pre-filled: the head adds into the master gradient
    loss, dx = ops.nmt_loss_head(x, k, dev(tgt_np), dev(lens_np), d_proj_kernel=dk, loss_scale=3.0)
    odt = torch.float64
    xo = torch.tensor(x_np, dtype=odt, requires_grad=True)
    ko = torch.tensor(k_np, dtype=odt, requires_grad=True)
    lo, _ = og.nmt_loss(xo, ko, torch.tensor(tgt_np), torch.tensor(lens_np))
    gx, gk = torch.autograd.grad(lo, [xo, ko])
    tol = TOL
    assert_close(loss, 3.0 * lo.detach().double().reshape(1), tol, "loss")
    assert_close(dx, 3.0 * gx.double(), tol, "dx")
    assert_close(dk - 1, 3.0 * gk.double(), tol, "d output_projection")
    for b in range(B):                                         # padded steps carry no gradient, exactly
        if lens_np[b] < T:
            assert float(dx[lens_np[b]:, b].abs().max()) == 0.0
    # forward only; a custom divisor (hparams.batch_size); an out-of-range label poisons the loss like TensorFlow's kernel
    l2, none = ops.nmt_loss_head(x, k, dev(tgt_np), dev(lens_np), need_dx=False, loss_batch_size=2 * B)
    assert none is None
    assert_close(l2, lo.detach().double().reshape(1) / 2, tol, "loss with another divisor")
    if lens_np[0] > 0:
        bad = tgt_np.copy(); bad[0, 0] = V
        l3, _ = ops.nmt_loss_head(x, k, dev(bad), dev(lens_np), need_dx=False)
        assert torch.isnan(l3).all()


def test_last_device_step_decoder_cells_then_loss():
    # the second device of the GNMT pipeline: decoder cells 1.., projection, loss; M micro-batches, K = 1 (F0 B0 F1 B1)
    from dapple_amd import ops
    L, U, B, T, V, M = 3, 32, 4, 6, 40, 2
    w_np = synthetic.gnmt_decoder_weights(61, 1, L, U, init_weight=0.3, perturb=True)
    r = np.random.Generator(np.random.PCG64(62))
    k_np = r.uniform(-0.3, 0.3, (U, V)).astype(np.float32)
    xs_np = [r.standard_normal((T, B, U)).astype(np.float32) for _ in range(M)]
    tg_np = [r.integers(0, V, (B, T)).astype(np.int32) for _ in range(M)]
    ln_np = [np.array([6, 2, 4, 1], np.int32), np.array([3, 6, 6, 5], np.int32)]
    st = runtime.gnmt_decoder_stage(L, U, B, T, stash_slots=1)
    st.bind(w_np)
    k = dev(k_np)
    dk = torch.zeros_like(k)
    losses, dxs = [], []
    for j in range(M):
        y = torch.empty(T, B, U, device="cuda")
        st.forward(0, dev(xs_np[j]), y)
        loss, dy = ops.nmt_loss_head(y, k, dev(tg_np[j]), dev(ln_np[j]), d_proj_kernel=dk)
        dx = torch.empty_like(y)
        st.backward(0, dy, dx)
        losses.append(loss); dxs.append(dx)
    st.sync()
    w_t = og.to_torch(w_np, torch.float64, requires_grad=True)
    ko = torch.tensor(k_np, dtype=torch.float64, requires_grad=True)
    names = sorted(w_t)
    acc = None
    for j in range(M):
        xo = torch.tensor(xs_np[j], dtype=torch.float64, requires_grad=True)
        lo, _ = og.nmt_loss(og.decoder_part2_forward(xo, None, w_t, 1, L), ko, torch.tensor(tg_np[j]), torch.tensor(ln_np[j]))
        gs = torch.autograd.grad(lo, [xo, ko] + [w_t[n] for n in names])
        assert_close(losses[j], lo.detach().reshape(1), TOL, "loss mb%d" % j)
        assert_close(dxs[j], gs[0], TOL, "input grad mb%d" % j)
        acc = list(gs[1:]) if acc is None else [a + g for a, g in zip(acc, gs[1:])]
    assert_close(dk, acc[0], TOL, "d output_projection")
    for n, g in zip(names, acc[1:]):
        if n.endswith("/kernel"):     # zero attention: compare the rows that carry a gradient, the others are exactly zero
            assert float(st.grads[n][U:2 * U].abs().max()) == 0.0
        assert_close(st.grads[n], g.reshape(st.grads[n].shape), TOL, "grad " + n)
    st.close()
