"""Classification block + loss of the last VGG19 stage (ds_vgg_head) through the C ABI against the fp64 oracle
(oracle/vgg.py::head_forward / head_loss), alone and behind the conv layers of the last device."""
import numpy as np
import pytest
import torch

from dapple_amd import ops, slices, synthetic
from oracle import vgg as ov
from util import assert_close, dev

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _case(B, Fe, Fc, Cl, seed, mode, labels=None):
    r = np.random.Generator(np.random.PCG64(seed))
    hw_np = synthetic.vgg_head_weights(seed, Fe, Fc, Cl, perturb=True)
    x_np = np.abs(r.standard_normal((B, Fe))).astype(np.float32)           # a pool output: non-negative
    lab = np.asarray(labels if labels is not None else r.integers(1, Cl, B), np.float32)
    hw = {k: dev(v) for k, v in hw_np.items()}
    g0 = {k: dev(r.standard_normal(v.shape).astype(np.float32)) for k, v in hw_np.items()}
    grads = {k: v.clone() for k, v in g0.items()}
    loss, probs, dx = ops.vgg_head(dev(x_np), hw, dev(lab), grads=grads, loss_mode=mode)
    torch.cuda.synchronize()
    return r, hw_np, x_np, lab, g0, grads, loss, probs, dx


@pytest.mark.parametrize("B,Fe,Fc,Cl", [(4, 36, 16, 8), (5, 200, 64, 12), (32, 25088, 4096, 1000)])
def test_sparse_cross_entropy_against_the_oracle(B, Fe, Fc, Cl):
    """Forward, loss and every gradient with the label as a class index; the last case is the reference's size
    (7 x 7 x 512 features, 4096 units, 1000 classes, micro-batch 32)."""
    r, hw_np, x_np, lab, g0, grads, loss, probs, dx = _case(B, Fe, Fc, Cl, 3 + B, "sparse_ce")
    w = ov.to_torch(hw_np, torch.float64, requires_grad=True)
    x = torch.tensor(x_np, dtype=torch.float64, requires_grad=True)
    p = ov.head_forward(x, w)
    ref = ov.head_loss(p, torch.tensor(lab), "sparse_ce")
    names = sorted(w)
    gr = torch.autograd.grad(ref, [x] + [w[n] for n in names])
    assert_close(probs, p.detach(), TOL, "probabilities")
    assert_close(loss, ref.detach().reshape(1), TOL, "loss")
    assert_close(dx, gr[0], TOL, "dx")
    for n, g in zip(names, gr[1:]):
        assert_close(grads[n] - g0[n], g, TOL, "gradient of %s (added to)" % n, floor=float(g0[n].abs().max()))


def test_loss_as_the_reference_writes_it():
    """K.categorical_crossentropy(x, label) with the softmax output in the target slot: the loss is -log(1 - 1e-7) in fp32
    arithmetic whatever the input, every gradient vanishes; a zero label is 0/0."""
    r, hw_np, x_np, lab, g0, grads, loss, probs, dx = _case(6, 72, 32, 12, 9, "as_written")
    w = ov.to_torch(hw_np, torch.float32)
    p = ov.head_forward(torch.tensor(x_np), w)
    ref = ov.head_loss(p, torch.tensor(lab), "as_written")                    # the oracle in fp32: the clip bound 1 - 1e-7 rounds to 1 - 2^-23
    assert abs(ref.item() - 1.1920929e-07) < 1e-12
    assert_close(probs, p, 1e-5, "probabilities")
    assert abs(loss.item() - ref.item()) <= 1e-5 * ref.item()
    assert float(dx.abs().max()) <= 1e-12
    for n in grads:
        assert float((grads[n] - g0[n]).abs().max()) <= 1e-6 * float(g0[n].abs().max()), n
    _, _, _, _, _, _, loss0, _, _ = _case(6, 72, 32, 12, 9, "as_written", labels=[3, 0, 2, 5, 1, 7])
    assert torch.isnan(loss0).all()


def test_rejects_bad_arguments():
    hw = {k: dev(v) for k, v in synthetic.vgg_head_weights(0, 8, 8, 8).items()}
    x = torch.zeros(2, 8, device="cuda")
    with pytest.raises(ValueError):
        ops.vgg_head(x, hw, torch.zeros(3, device="cuda"))
    with pytest.raises(ValueError):
        ops.vgg_head(x, hw, torch.zeros(2, device="cuda"), loss_mode="mse")
    with pytest.raises(ValueError):
        ops.vgg_head(torch.zeros(2, 12, device="cuda"), hw, torch.zeros(2, device="cuda"))
    with pytest.raises(Exception):                                        # a label that is no class index: NaN loss, no error
        loss, _, _ = ops.vgg_head(x, hw, torch.tensor([1.0, 9.0], device="cuda"), loss_mode="sparse_ce")
        assert not torch.isnan(loss).any()


def test_last_device_of_the_sliced_model():
    """SliceVGG19(local_device=1): block5_conv3, block5_conv4, block5_pool, the classification block and the loss, then the
    backward pass down to the boundary activation - against autograd through the oracle's conv stack + head."""
    B, Hh, Ww, Cin, Cl, Fc = 4, 4, 4, 32, 12, 32
    layers = [("block5_conv3", 32), ("block5_conv4", 32), ("block5_pool", None)]
    r = np.random.Generator(np.random.PCG64(21))
    wv = synthetic.vgg_weights(5, layers, Cin, perturb=True)
    wv.update(synthetic.vgg_head_weights(6, 2 * 2 * 32, Fc, Cl, perturb=True))
    m = slices.SliceVGG19(num_replica=15, classes=Cl, weight_values=wv, local_device=1, loss_mode="sparse_ce", fc_units=Fc)
    m.layers = layers                                                    # the reference's 512 channels cut to 32 for the CPU oracle
    x_np = r.standard_normal((B, Hh, Ww, Cin)).astype(np.float32)
    lab = r.integers(0, Cl, B)
    loss, outs = m.build(dev(x_np), lab.reshape(B, 1))
    assert outs[1] is loss and tuple(outs[0].shape) == (B, Hh, Ww, Cin)
    d_in = torch.empty(B, Hh, Ww, Cin, device="cuda")
    m.backward(d_in)
    m.stage.sync()
    w = ov.to_torch(wv, torch.float64, requires_grad=True)
    x = torch.tensor(x_np, dtype=torch.float64, requires_grad=True)
    y = ov.stage_forward(x, w, layers)
    ref = ov.head_loss(ov.head_forward(y.reshape(B, -1), w), torch.tensor(lab), "sparse_ce")
    names = sorted(w)
    gr = dict(zip(names, torch.autograd.grad(ref, [w[n] for n in names] + [x])))
    gx = torch.autograd.grad(ov.head_loss(ov.head_forward(ov.stage_forward(x, w, layers).reshape(B, -1), w), torch.tensor(lab), "sparse_ce"), x)[0]
    assert_close(loss, ref.detach().reshape(1), TOL, "loss")
    assert_close(d_in, gx, TOL, "gradient of the boundary activation")
    for n in names:
        got = m.head_grads[n] if n.startswith(("fc1/", "fc2/", "predictions/")) else m.stage.grads[n]
        assert_close(got, gr[n], TOL, "gradient of " + n)
    with pytest.raises(ValueError):
        m.backward()                                                     # nothing pending
    m.stage.close()
