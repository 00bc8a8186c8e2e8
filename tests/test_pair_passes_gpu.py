"""F(j+1) and B(j) as one call (ds_stage_forward_backward): a BERT stage in the benchmarked mode walks both chains
together, one grouped launch per level.  Same results as the separate calls, against the oracle and against each other."""
import pytest
import torch

from dapple_amd import runtime, synthetic
from test_stage_bert_gpu import run_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("overlap", [False, True])
@pytest.mark.parametrize("use_mask", [False, True])
def test_paired_passes_against_the_oracle(overlap, use_mask):
    # hidden 256 = 4 heads of 64, 5 micro-batches: the last weight-gradient group is short, the last backward pass alone
    run_case("bf16", 2, 256, 4, 512, 2, 128, 5, use_mask=use_mask, wgrad_group=4, overlap=overlap, pair_passes=True)
    run_case("bf16", 3, 256, 4, 1024, 1, 64, 6, use_mask=use_mask, wgrad_group=2, overlap=overlap, pair_passes=True, K=3)


def test_paired_passes_at_the_benchmark_layer_shape():
    c = synthetic.CONFIGS["bert48_half"]
    run_case("bf16", 2, c["hidden"], c["heads"], c["ffn"], c["micro_batch"], c["seq"], 4, stddev=0.02, perturb=False, seed=c["index"],
             wgrad_group=4, overlap=True, pair_passes=True, odtype=torch.float32)


def test_paired_passes_equal_separate_passes_over_steps():
    """Three steps in a row (stash positions and operand ring wrap), paired and separate calls, one stream and three:
    outputs and input gradients agree to bf16 rounding of a different tile order, weight gradients likewise."""
    L, H, N, F, B, S, M = 2, 256, 4, 512, 2, 128, 6
    w = synthetic.bert_weights(21, L, H, F)
    xs = [torch.as_tensor(x).cuda().bfloat16() for x in synthetic.bert_activation_inputs(22, M, B, S, H)]
    dys = [torch.as_tensor(x).cuda().bfloat16() for x in synthetic.upstream_grads(23, M, (B * S, H))]
    res = []
    for pair, overlap in ((False, True), (True, True), (True, False), (True, True)):
        st = runtime.bert_stage(L, H, N, F, B, S, "bf16", stash_slots=2, wgrad_group=4)
        st.bind(w)
        if overlap:
            st.enable_overlap()
        outs = [torch.empty(B * S, H, dtype=torch.bfloat16, device="cuda") for _ in range(M)]
        dxs = [torch.empty_like(o) for o in outs]
        rt = runtime.StageRuntime(st, 0, 2, M, pair_passes=pair)
        for _ in range(3):
            st.refresh_weights()
            st.zero_grads()
            rt.step(xs, dys, outs, dxs)
        st.sync()
        res.append(([o.float().cpu() for o in outs], [d.float().cpu() for d in dxs], {k: v.cpu().clone() for k, v in st.grads.items()}))
        st.close()
    # paired runs are bit-identical to each other whatever the streams (atomics aside: LayerNorm and bias gradients)
    for a, b in zip(res[1][0] + res[1][1], res[2][0] + res[2][1]):
        assert torch.equal(a, b)
    for a, b in zip(res[1][0] + res[1][1], res[3][0] + res[3][1]):
        assert torch.equal(a, b)
    for other in res[1:]:
        for a, b in zip(res[0][0] + res[0][1], other[0] + other[1]):
            assert float((a - b).abs().max()) <= 2e-2 * float(a.abs().max())
        for k in res[0][2]:
            a, b = res[0][2][k], other[2][k]
            scale = float(a.abs().max())
            if k.endswith("/key/bias"):
                scale = float(res[0][2][k.replace("/key/", "/query/")].abs().max())
            assert float((a - b).abs().max()) <= 2e-2 * scale + 1e-12, k


def test_paired_call_checks_its_slots():
    st = runtime.bert_stage(1, 256, 4, 512, 1, 64, "bf16", stash_slots=2, wgrad_group=2)
    st.bind(synthetic.bert_weights(5, 1, 256, 512))
    x = torch.zeros(64, 256, dtype=torch.bfloat16, device="cuda")
    y, d, dx = torch.empty_like(x), torch.zeros_like(x), torch.empty_like(x)
    with pytest.raises(Exception):      # nothing forwarded into slot 1 yet
        st.forward_backward(0, x, y, 1, d, dx)
    st.forward(1, x, y)
    with pytest.raises(Exception):      # one slot for both
        st.forward_backward(1, x, y, 1, d, dx)
    st.forward_backward(0, x, y, 1, d, dx)
    st.backward(0, d, dx)
    st.sync()
    st.close()
