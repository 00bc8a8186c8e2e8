"""Pins of oracle/optim.py (CPU): the reference's own known-answer test, hand-computed steps, a library
routine and brute force."""
import numpy as np
import torch

from oracle import optim as oo


def test_reference_known_answer_adam_weight_decay():
    # bert/models/bert/optimization_test.py:25-44: w0 = [0.1,-0.2,-0.1], loss = mean((x - w)^2), lr 0.2, 100 steps
    x = np.array([0.4, 0.2, -0.5])
    p = {"w": np.array([0.1, -0.2, -0.1])}
    opt = oo.AdamWeightDecay(learning_rate=0.2)
    for _ in range(100):
        g = -2.0 * (x - p["w"]) / 3.0            # d/dw mean((x-w)^2)
        opt.apply_gradients({"w": g}, p)
    np.testing.assert_allclose(p["w"], x, rtol=1e-2, atol=1e-2)


def test_first_step_closed_form_and_decay_exclusion():
    # zero moments: m = (1-b1) g, v = (1-b2) g^2, update = m / (sqrt(v) + eps) [+ wd * w]
    g = np.array([0.5, -2.0, 0.0])
    w0 = np.array([1.0, -1.0, 3.0])
    for name, decayed in (("layer_0/output/dense/kernel", True), ("layer_0/output/LayerNorm/gamma", False),
                          ("layer_0/output/dense/bias", False)):
        p = {name: w0.copy()}
        opt = oo.AdamWeightDecay(0.1, weight_decay_rate=0.01, exclude_from_weight_decay=["LayerNorm", "layer_norm", "bias"])
        opt.apply_gradients({name: g}, p)
        upd = 0.1 * g / (np.sqrt(0.001) * np.abs(g) + 1e-6) + (0.01 * w0 if decayed else 0.0)
        np.testing.assert_allclose(p[name], w0 - 0.1 * upd, rtol=1e-12)
    # a dropped (1-b1) or a sign error changes the first element by > 10 %
    assert abs((w0 - 0.1 * upd)[0] - w0[0]) > 0.1


def test_adam_matches_library_routine():
    # tf.train.AdamOptimizer == torch.optim.Adam up to the epsilon placement; with eps -> 0 they coincide
    r = np.random.default_rng(0)
    w0 = r.standard_normal(7)
    p = {"w": w0.copy()}
    tw = torch.tensor(w0, dtype=torch.float64, requires_grad=True)
    topt = torch.optim.Adam([tw], lr=0.05, betas=(0.9, 0.999), eps=1e-300)
    opt = oo.Adam(0.05, epsilon=1e-300)
    for i in range(5):
        g = r.standard_normal(7)
        opt.apply_gradients({"w": g}, p)
        tw.grad = torch.tensor(g)
        topt.step()
    np.testing.assert_allclose(p["w"], tw.detach().numpy(), rtol=1e-10)


def test_clip_by_global_norm_brute_force():
    r = np.random.default_rng(1)
    grads = [r.standard_normal((3, 4)), r.standard_normal(5)]
    flat = np.concatenate([g.ravel() for g in grads])
    norm = float(np.sqrt((flat ** 2).sum()))
    clipped, n = oo.clip_by_global_norm(grads, 1.0)
    assert abs(n - norm) < 1e-12
    np.testing.assert_allclose(np.concatenate([c.ravel() for c in clipped]), flat / norm, rtol=1e-12)
    assert abs(oo.global_norm(clipped) - 1.0) < 1e-12
    same, _ = oo.clip_by_global_norm(grads, 100.0)          # below the threshold: untouched
    np.testing.assert_array_equal(np.concatenate([c.ravel() for c in same]), flat)


def test_gradient_descent_and_xlnet_schedule():
    p = {"w": np.array([1.0, 2.0])}
    oo.gradient_descent({"w": np.array([10.0, -10.0])}, p, 0.1)
    np.testing.assert_allclose(p["w"], [0.0, 3.0])
    # xlnet_utils.py:179-193 with run.sh-like numbers: warm-up is linear in the step, decay is linear to the floor
    lr, wu, ts, ratio = 1e-4, 500, 4000, 0.1
    assert oo.xlnet_learning_rate(250, lr, wu, ts, ratio) == 0.5 * lr
    assert abs(oo.xlnet_learning_rate(1000, lr, wu, ts, ratio) - ((lr - lr * ratio) * (1 - 500 / 3500) + lr * ratio)) < 1e-18
    assert abs(oo.xlnet_learning_rate(10 ** 6, lr, wu, ts, ratio) - lr * ratio) < 1e-18
    from dapple_amd import optim
    for s in (0, 250, 999, 1000, 2500, 4000, 9999):
        assert optim.xlnet_learning_rate(s, lr, wu, ts, ratio) == oo.xlnet_learning_rate(s, lr, wu, ts, ratio)
