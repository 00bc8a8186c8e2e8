"""Fused clip + optimizer kernels against the CPU oracle through the C ABI (fp32, 1e-5 relative), the
reference's known-answer test on the GPU, and a stage step -> apply -> refresh -> forward round trip."""
import numpy as np
import pytest
import torch

from dapple_amd import optim, runtime, synthetic
from oracle import bert as ob
from oracle import optim as oo
from util import assert_close

pytestmark = pytest.mark.gpu
EXCLUDE = ["LayerNorm", "layer_norm", "bias"]


def make_params(seed):
    r = np.random.default_rng(seed)
    shapes = {"layer_0/dense/kernel": (37, 53), "layer_0/dense/bias": (53,), "layer_0/LayerNorm/gamma": (53,),
              "big/kernel": (300, 129), "odd/kernel": (3,), "one/bias": (1,)}      # ragged tails, several chunks
    return {n: r.standard_normal(s).astype(np.float32) for n, s in shapes.items()}, r


def test_reference_known_answer_on_gpu():
    # bert/models/bert/optimization_test.py:25-44
    x = torch.tensor([0.4, 0.2, -0.5], device="cuda")
    fp = optim.FlatParams({"w": np.array([0.1, -0.2, -0.1], np.float32)})
    opt = optim.AdamWeightDecayOptimizer(learning_rate=0.2)
    for _ in range(100):
        fp.grads["w"].copy_(-2.0 * (x - fp.weights["w"]) / 3.0)
        opt.apply_gradients(fp)
    np.testing.assert_allclose(fp.weights["w"].cpu().numpy(), [0.4, 0.2, -0.5], rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("clip", [None, 0.5, 1e6])
def test_adam_weight_decay_matches_oracle(clip):
    w, r = make_params(3)
    fp = optim.FlatParams(w)
    p = {n: a.astype(np.float64) for n, a in w.items()}
    opt = optim.AdamWeightDecayOptimizer(3e-3, weight_decay_rate=0.01, beta_1=0.9, beta_2=0.999, epsilon=1e-6,
                                         exclude_from_weight_decay=EXCLUDE)
    ref = oo.AdamWeightDecay(3e-3, weight_decay_rate=0.01, exclude_from_weight_decay=EXCLUDE)
    for _ in range(4):
        g = {n: r.standard_normal(a.shape).astype(np.float32) for n, a in w.items()}
        for n in g:
            fp.grads[n].copy_(torch.as_tensor(g[n]))
        opt.apply_gradients(fp, max_gradient_norm=clip)
        gl = [g[n] for n in g]
        if clip is not None:
            gl, _ = oo.clip_by_global_norm(gl, clip)
        ref.apply_gradients(dict(zip(g, gl)), p)
    for n in w:
        assert_close(fp.weights[n], p[n], 1e-5, "weights " + n)
    m, v = opt.moments(fp)
    off, k = fp.weight_offsets[3], fp.weight_numels[3]
    assert_close(m[off:off + k], ref.m["big/kernel"].ravel(), 1e-5, "adam_m")
    assert_close(v[off:off + k], ref.v["big/kernel"].ravel(), 1e-5, "adam_v")


def test_adam_and_sgd_match_oracle():
    w, r = make_params(5)
    for kind in ("adam", "sgd"):
        fp = optim.FlatParams(w)
        p = {n: a.astype(np.float64) for n, a in w.items()}
        opt = optim.AdamOptimizer(1e-2, epsilon=1e-8) if kind == "adam" else optim.GradientDescentOptimizer(0.1)
        ref = oo.Adam(1e-2, epsilon=1e-8)
        for step in range(3):
            g = {n: r.standard_normal(a.shape).astype(np.float32) for n, a in w.items()}
            for n in g:
                fp.grads[n].copy_(torch.as_tensor(g[n]))
            opt.apply_gradients(fp, max_gradient_norm=2.0)
            gl, _ = oo.clip_by_global_norm([g[n] for n in g], 2.0)
            if kind == "adam":
                ref.apply_gradients(dict(zip(g, gl)), p)
            else:
                oo.gradient_descent(dict(zip(g, gl)), p, 0.1)
        for n in w:
            assert_close(fp.weights[n], p[n], 1e-5, kind + " weights " + n)


def test_padding_between_tensors_is_left_alone():
    w, r = make_params(7)
    fp = optim.FlatParams(w)
    fp.flat_weights.fill_(7.0)
    fp.flat_grads.fill_(1.0)
    optim.GradientDescentOptimizer(1.0).apply_gradients(fp)
    mask = torch.zeros_like(fp.flat_weights, dtype=torch.bool)
    for off, k in zip(fp.weight_offsets, fp.weight_numels):
        mask[off:off + k] = True
    assert torch.all(fp.flat_weights[mask] == 6.0) and torch.all(fp.flat_weights[~mask] == 7.0)


def test_clip_by_global_norm_over_several_parameter_sets():
    """tf.clip_by_global_norm runs over the gradients of all slices (bert/graph.py:162-165): two parameter sets given
    as a list share one norm and one factor; given one by one each would get its own."""
    wa, r = make_params(11)
    wb = {"head/output_weights": r.standard_normal((2, 40)).astype(np.float32), "head/output_bias": r.standard_normal(2).astype(np.float32)}
    fa, fb = optim.FlatParams(wa), optim.FlatParams(wb)
    ga = {n: (r.standard_normal(a.shape) * 3).astype(np.float32) for n, a in wa.items()}
    gb = {n: (r.standard_normal(a.shape) * 0.05).astype(np.float32) for n, a in wb.items()}
    for fp, g in ((fa, ga), (fb, gb)):
        for n in g:
            fp.grads[n].copy_(torch.as_tensor(g[n]))
    clip = 0.75
    opt = optim.GradientDescentOptimizer(0.5)
    opt.apply_gradients([fa, fb], max_gradient_norm=clip)
    names = list(ga) + list(gb)
    clipped, norm = oo.clip_by_global_norm([ga[n] for n in ga] + [gb[n] for n in gb], clip)
    assert norm > clip * 4          # the clip is active, and set b alone would not have been clipped at all
    assert np.sqrt(sum(float((g.astype(np.float64) ** 2).sum()) for g in gb.values())) < clip
    ref = dict(zip(names, clipped))
    for fp, w in ((fa, wa), (fb, wb)):
        for n in w:
            assert_close(fp.weights[n], w[n].astype(np.float64) - 0.5 * ref[n], 1e-5, "sgd under the global clip: " + n)


def test_stage_step_apply_refresh_forward():
    # one training step of a BERT stage: accumulate over M micro-batches, clip, AdamWeightDecay, refresh; the next
    # forward must equal the oracle's forward with the oracle-updated weights
    L, H, N, F, B, S, M = 2, 64, 4, 128, 2, 16, 3
    w = synthetic.bert_weights(21, L, H, F)
    xs_np = synthetic.bert_activation_inputs(22, M, B, S, H)
    dys_np = synthetic.upstream_grads(23, M, (B * S, H))
    st = runtime.bert_stage(L, H, N, F, B, S, "fp32", stash_slots=2)
    st.bind(w)
    xs = [torch.as_tensor(x).cuda() for x in xs_np]
    dys = [torch.as_tensor(d).cuda() for d in dys_np]
    outs = [torch.empty(B * S, H, device="cuda") for _ in range(M)]
    dxs = [torch.empty_like(o) for o in outs]
    rt = runtime.StageRuntime(st, 0, 2, M)
    rt.step(xs, dys, outs, dxs)
    opt = optim.AdamWeightDecayOptimizer(1e-3, weight_decay_rate=0.01, exclude_from_weight_decay=EXCLUDE)
    opt.apply_gradients(st, max_gradient_norm=1.0)     # marks the stage: its next forward pass rebuilds the compute copies
    st.zero_grads()
    rt.step(xs, dys, outs, dxs)
    st.sync()
    # oracle
    wt = ob.to_torch(w, torch.float64, requires_grad=True)
    acc = {}
    for j in range(M):
        _, _, dw = ob.stage_vjp(torch.as_tensor(xs_np[j]).double(), wt, torch.as_tensor(dys_np[j]).double(), list(range(L)), B, S, N)
        for k, g in dw.items():
            acc[k] = g.clone() if k not in acc else acc[k] + g
    names = list(acc)
    clipped, _ = oo.clip_by_global_norm([acc[k].numpy() for k in names], 1.0)
    p = {k: np.asarray(w[k], np.float64).copy() for k in names}
    oo.AdamWeightDecay(1e-3, weight_decay_rate=0.01, exclude_from_weight_decay=EXCLUDE).apply_gradients(dict(zip(names, clipped)), p)
    for k in names:
        if k.endswith("/key/bias"):
            # softmax is invariant to the key bias: its gradient is rounding noise, which Adam's normalisation
            # amplifies differently in fp32 and fp64 (and which cannot change any output)
            continue
        # biases start at zero, so the update IS the value: it carries the stage gradients' 1e-4 tolerance
        assert_close(st.weights[k], p[k].reshape(st.weights[k].shape), 1e-4, "updated " + k)
    w2 = ob.to_torch({k: p[k] for k in names}, torch.float64, requires_grad=True)
    o2, _, _ = ob.stage_vjp(torch.as_tensor(xs_np[0]).double(), w2, torch.as_tensor(dys_np[0]).double(), list(range(L)), B, S, N)
    assert_close(outs[0], o2, 1e-4, "forward after the update")
    st.close()
