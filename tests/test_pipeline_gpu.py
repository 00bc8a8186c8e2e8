"""All stages of a sliced BERT on one GPU under the unrolled early-backward graph (bert/graph.py:97-161): losses,
boundary tensors and the accumulated gradients of every stage and of the head against autograd through the whole model."""
import numpy as np
import pytest
import torch

from dapple_amd import ops, runtime, synthetic
from oracle import bert as ob
from oracle import head as oh
from util import assert_close, dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("overlap", [False, True])
@pytest.mark.parametrize("split,M", [((1, 2, 1), 5), ((2, 2), 3), ((4,), 2)])
def test_whole_model_pipeline_matches_autograd(split, M, overlap):
    """overlap: every stage runs its backward passes on streams of its own; the gradient handed from stage to stage then
    travels with the event of the pass that wrote it."""
    H, N, F, B, S, V = 64, 4, 128, 2, 16, 50
    L = sum(split)
    emb = (V, 2, 32)
    w_np = synthetic.bert_weights(51, L, H, F, embeddings=emb, stddev=0.05, perturb=True)
    r = np.random.default_rng(52)
    hw_np, hb_np = r.standard_normal((2, H)) * 0.05, r.standard_normal(2) * 0.05
    ids_np = synthetic.bert_id_inputs(53, M, B, S, V)
    sp_np = r.integers(0, S, (M, B)).astype(np.int32)
    ep_np = r.integers(0, S, (M, B)).astype(np.int32)
    nst = len(split)
    stages, first = [], 0
    for i, n in enumerate(split):
        st = runtime.bert_stage(n, H, N, F, B, S, "fp32", stash_slots=runtime.stash_depth(i, nst),
                                embeddings=emb if i == 0 else None, first_layer=first, wgrad_group=2 if i == 0 else 1)
        st.bind(w_np)
        if overlap:
            assert st.overlap_supported()
            st.enable_overlap()
        stages.append(st)
        first += n
    hw, hb = dev(hw_np, torch.float32), dev(hb_np, torch.float32)
    dhw, dhb = torch.zeros_like(hw), torch.zeros_like(hb)
    sp, ep = [dev(x) for x in sp_np], [dev(x) for x in ep_np]

    def loss_fn(j, out):
        loss, _, _, dx = ops.squad_head(out.reshape(B * S, H), B, S, hw, hb, sp[j], ep[j], dhw, dhb)
        return loss, dx

    pipe = runtime.PipelineRuntime(stages, M, loss_fn)
    losses = pipe.step([dev(x) for x in ids_np])
    torch.cuda.synchronize()
    # every stage issued its own early-backward order, and nothing ran before its data existed
    for i in range(nst):
        assert [(op, j) for (s, op, j) in pipe.issued if s == i] == runtime.schedule_ops(i, nst, M)
    seen = set()
    for s, op, j in pipe.issued:
        if op == "F":
            assert s == 0 or (s - 1, "F", j) in seen
        else:
            assert (s, "F", j) in seen and (s == nst - 1 or (s + 1, "B", j) in seen)
        seen.add((s, op, j))
    # oracle: the un-sliced model, one autograd pass per micro-batch, gradients summed (tf.accumulate_n)
    w_t = ob.to_torch(w_np, torch.float64, requires_grad=True)
    hw_t = torch.as_tensor(hw_np).double().requires_grad_(True)
    hb_t = torch.as_tensor(hb_np).double().requires_grad_(True)
    names = sorted(w_t)
    acc = None
    for j in range(M):
        x = ob.stage_forward(torch.as_tensor(ids_np[j]), w_t, list(range(L)), B, S, N)
        lo, _, _ = oh.squad_loss(x.reshape(B, S, H), hw_t, hb_t, torch.as_tensor(sp_np[j]), torch.as_tensor(ep_np[j]))
        assert_close(losses[j], lo.reshape(1), 1e-4, "loss mb%d" % j)
        assert_close(pipe.all_outputs[j][-1], x.reshape(-1), 1e-4, "last boundary tensor mb%d" % j)
        g = torch.autograd.grad(lo, [w_t[n] for n in names] + [hw_t, hb_t], allow_unused=True)
        acc = list(g) if acc is None else [a + b if b is not None else a for a, b in zip(acc, g)]
    ref = dict(zip(names, acc[:-2]))
    for st in stages:
        for n in st.weight_names:
            floor = ref[n.replace("/key/", "/query/")].abs().max().item() if n.endswith("/key/bias") else None
            if n == "bert/encoder/layer_%d/output/LayerNorm/beta" % (L - 1):
                # the head's input gradient sums to zero over the sequence (softmax minus one-hot), so this one
                # vanishes identically: judge it on the scale of gamma's gradient
                floor = ref[n.replace("beta", "gamma")].abs().max().item()
            assert_close(st.grads[n], ref[n], 1e-4, "accumulated grad " + n, floor=floor)
    assert_close(dhw, acc[-2], 1e-4, "head weights")
    assert_close(dhb, acc[-1], 1e-4, "head bias", floor=float(acc[-2].abs().max()))
    for st in stages:
        st.close()


def test_backward_waits_for_upstream_gradient_produced_on_the_stage_stream():
    """Forward/backward overlap on: the upstream gradient of a pass is written by kernels queued on the stage's stream
    AFTER that micro-batch's forward pass (a loss head), with the next forward pass queued behind them.  Both ways of
    saying when it is ready - ds_stage_backward (everything queued so far) and ds_stage_backward_after (an event behind
    the producer) - give the one-stream result bit for bit."""
    L, H, N, F, B, S, M = 2, 256, 4, 1024, 2, 128, 4
    w_np = synthetic.bert_weights(61, L, H, F, stddev=0.05, perturb=True)
    xs = [dev(x, torch.bfloat16) for x in synthetic.bert_activation_inputs(62, M, B, S, H)]
    seed = [dev(x, torch.bfloat16) for x in synthetic.upstream_grads(63, M, (B * S, H))]

    def run(mode):
        st = runtime.bert_stage(L, H, N, F, B, S, "bf16", stash_slots=2)
        st.bind(w_np)
        if mode != "one stream":
            st.enable_overlap()
        outs = [torch.empty(B * S, H, dtype=torch.bfloat16, device="cuda") for _ in range(M)]
        dxs = [torch.empty_like(o) for o in outs]
        douts = [torch.full_like(o, float("nan")) for o in outs]
        slot_of, free = {}, [0, 1]

        def produce(j):   # a slow elementwise chain standing in for a loss head: d_out = f(out, seed)
            t = outs[j].float()
            for _ in range(40):
                t = t * 0.999 + 0.001
            douts[j].copy_(t.to(torch.bfloat16) * 0.01 + seed[j])
            ev = torch.cuda.Event()
            ev.record()
            return ev

        evs = {}
        for op, j in runtime.schedule_ops(0, 2, M):
            if op == "F":
                slot_of[j] = free.pop(0)
                st.forward(slot_of[j], xs[j], outs[j])
                evs[j] = produce(j)
            else:
                st.backward(slot_of[j], douts[j], dxs[j], ready=evs[j] if mode == "event" else False)
                free.append(slot_of.pop(j))
        st.sync()
        res = ([d.clone() for d in dxs], {n: g.clone() for n, g in st.grads.items()})
        st.close()
        return res

    ref_dx, ref_g = run("one stream")
    for mode in ("queued so far", "event"):
        dx, g = run(mode)
        for j in range(M):
            assert torch.equal(dx[j], ref_dx[j]), "%s: input gradient of micro-batch %d" % (mode, j)
        for n in ref_g:
            # LayerNorm / bias gradients are fp32 atomic sums whose order is not fixed: compare those at rounding level
            if n.endswith(("kernel",)):
                assert torch.equal(g[n], ref_g[n]), "%s: %s" % (mode, n)
            else:
                # (the key bias gradient is zero up to what two fp32 sums of the same terms differ by: judged on the query bias's scale)
                scale = float(ref_g[n.replace("/key/bias", "/query/bias")].abs().max()) + 1e-30
                assert float((g[n] - ref_g[n]).abs().max()) <= 1e-5 * scale, "%s: %s" % (mode, n)


def test_pipeline_rejects_mismatched_stages():
    a = runtime.bert_stage(1, 64, 4, 128, 2, 16, "fp32", stash_slots=2)
    b = runtime.bert_stage(1, 32, 4, 64, 2, 16, "fp32", stash_slots=1)
    with pytest.raises(ValueError, match="hands over"):
        runtime.PipelineRuntime([a, b], 2, lambda j, out: (None, out))
    with pytest.raises(ValueError, match="stash slots"):
        runtime.PipelineRuntime([b, b], 2, lambda j, out: (None, out))
    a.close()
    b.close()
