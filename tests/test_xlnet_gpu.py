"""XLNet stage parity through the C ABI against the CPU oracle: the reference form (content stream, no
memory), then memory and the query stream.  fp32 1e-4, bf16 2e-2 relative."""
import numpy as np
import pytest
import torch

from dapple_amd import runtime, synthetic
from oracle import xlnet as ox
from util import assert_close, dev

pytestmark = pytest.mark.gpu
TOL = {"fp32": 1e-4, "bf16": 2e-2}
ADT = {"fp32": torch.float32, "bf16": torch.bfloat16}


def run_case(dtype, L, H, N, F, B, Q, Mm, S, M, K=2, seed=0, use_seg=True, mask_kind="perm", stddev=0.1, perturb=True,
             odtype=torch.float64, overlap=False, fused=False):
    adt = ADT[dtype]
    klen = Mm + Q
    w_np = synthetic.xlnet_weights(synthetic.SEED_WEIGHT + seed, L, H, N, F, stddev=stddev, perturb=perturb)
    xs_np = synthetic.xlnet_stream_inputs(synthetic.SEED_INPUT + seed, M, Q, B, H, streams=S)
    dys_np = synthetic.xlnet_stream_inputs(synthetic.SEED_GRAD + seed, M, Q, B, H, streams=S)
    mems_np = synthetic.xlnet_mems(50 + seed, L, Mm, B, H) if Mm else None
    r = np.random.Generator(np.random.PCG64(70 + seed))
    seg_ids = (r.random((Q, B)) > 0.6).astype(np.int64) if use_seg else np.zeros((Q, B), np.int64)
    if mask_kind == "perm":
        masks_np = list(synthetic.xlnet_perm_masks(90 + seed, Q, Mm, B))[:S]
    elif mask_kind == "input":       # the reference's mask: padding keys masked except on the diagonal
        im = (r.random((B, Q)) > 0.7).astype(np.int64)
        masks_np = [ox.attn_mask_from_input_mask(torch.from_numpy(im), Mm).numpy().astype(np.float32)] * S
    else:
        masks_np = None

    stage = runtime.xlnet_stage(L, H, N, F, B, Q, dtype, stash_slots=K, mem_len=Mm, streams=S, fused_attention=fused)
    stage.bind(w_np)
    if overlap:
        stage.enable_overlap()     # backward passes on the handle's second stream
    xs = [dev(np.stack(x), adt) for x in xs_np]
    dys = [dev(np.stack(d), adt) for d in dys_np]
    outs = [torch.empty(S, Q, B, H, dtype=adt, device="cuda") for _ in range(M)]
    dxs = [torch.empty_like(o) for o in outs]
    masks = None if masks_np is None else dev(np.stack(masks_np))
    seg_mat_t = ox.seg_mat_from_ids(torch.from_numpy(seg_ids), Mm)
    seg_mat = dev(seg_mat_t.numpy().astype(np.uint8)) if use_seg else None
    mems = None if mems_np is None else dev(np.stack(mems_np), adt)
    rt = runtime.StageRuntime(stage, 0, K, M)
    rt.step(xs, dys, outs, dxs, before_forward=lambda slot, j: stage.set_inputs(slot, masks, seg_mat, mems))
    stage.sync()

    w_t = ox.to_torch(w_np, odtype, requires_grad=True)
    mems_o = None if mems is None else [m.to(odtype) for m in mems.cpu()]
    masks_o = [torch.zeros(Q, klen, B, dtype=odtype)] * S if masks_np is None else [torch.from_numpy(m).to(odtype) for m in masks_np]
    acc = {}
    tol = TOL[dtype]
    for j in range(M):
        streams = [xs[j][s].cpu().to(odtype) for s in range(S)]
        d_outs = [dys[j][s].cpu().to(odtype) for s in range(S)]
        o, dx, dw = ox.stage_vjp(streams, mems_o, w_t, d_outs, list(range(L)), N, masks_o, torch.from_numpy(seg_ids))
        for s in range(S):
            assert_close(outs[j][s], o[s], tol, "output mb%d stream%d" % (j, s))
            assert_close(dxs[j][s], dx[s], tol, "input grad mb%d stream%d" % (j, s))
        for n_, g in dw.items():
            acc[n_] = g.clone() if n_ not in acc else acc[n_] + g
    for n_ in stage.weight_names:
        # with a single segment the segment term is the same for every key of a row, so softmax cancels it
        # and the gradients of bias_segment / seg_emb vanish identically: judge them against the size of the
        # bias_context gradient instead of against rounding noise
        floor = None
        if not use_seg and n_.endswith(("bias_segment", "seg_emb")):
            floor = acc[n_.rsplit("/", 1)[0] + "/bias_context"].abs().max().item()
        want = acc[n_].reshape(stage.grads[n_].shape)
        if use_seg and n_.endswith("bias_segment") and dtype == "bf16":
            # Each row's two segment-score gradients cancel (a softmax row's score gradients sum to zero), so this
            # gradient is a small difference - 10 to 40 times below the two sibling biases added to the same q - and
            # carries the rounding of the bf16 probabilities at their scale, not its own: judged on a tenth of
            # bias_context's scale where its own maximum is smaller than that.
            sib = 0.1 * acc[n_.rsplit("/", 1)[0] + "/bias_context"].abs().max().item()
            if want.abs().max().item() < sib:
                err = (stage.grads[n_].double().cpu() - want).abs().max().item() / sib
                assert err <= tol, "accumulated grad %s: %.3e of a tenth of the bias_context scale > tol %.1e" % (n_, err, tol)
                continue
        assert_close(stage.grads[n_], want, tol, "accumulated grad " + n_, floor=floor)
    stage.close()


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_reference_form_content_stream_no_memory(dtype):
    run_case(dtype, L=2, H=64, N=4, F=128, B=2, Q=16, Mm=0, S=1, M=3, mask_kind="input")


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_memory_and_two_streams(dtype):
    run_case(dtype, L=2, H=64, N=4, F=128, B=2, Q=16, Mm=8, S=2, M=2, seed=1)


def test_no_masks_no_segments_single_layer_fp32():
    run_case("fp32", L=1, H=32, N=2, F=64, B=1, Q=8, Mm=8, S=2, M=1, K=1, seed=2, use_seg=False, mask_kind=None)


def test_config4_shape_one_layer_bf16():
    # BASELINE configs[4] at its real layer shape (seq 512 + memory 384, hidden 1024, 16 heads, two streams), depth 1
    c = synthetic.CONFIGS["xlnet36_half"]
    run_case("bf16", 1, c["hidden"], c["heads"], c["ffn"], c["micro_batch"], c["seq"], c["mem_len"], c["streams"], M=1, K=1,
             seed=c["index"], stddev=0.02, perturb=False, odtype=torch.float32)


@pytest.mark.parametrize("Q,Mm,S,B,mask_kind,use_seg", [(64, 32, 2, 2, "perm", True), (128, 0, 1, 1, "input", True),
                                                         (64, 96, 2, 1, "perm", False), (64, 0, 1, 2, None, True)])
def test_fused_forward_attention_shapes(Q, Mm, S, B, mask_kind, use_seg):
    # the forward attention as one kernel (scores, relative shift, softmax, P V, probabilities for the backward pass),
    # an option of the stage for head size 64 and seq a multiple of 64; key counts of 96, 128, 160 and 64 cover partial
    # and single chunks; the permutation masks include rows whose keys in a 32-key step are all masked
    run_case("bf16", L=2, H=128, N=2, F=256, B=B, Q=Q, Mm=Mm, S=S, M=2, K=1, seed=11 + Q + Mm, use_seg=use_seg, mask_kind=mask_kind,
             fused=True)


def test_fused_forward_attention_config4_shape():
    c = synthetic.CONFIGS["xlnet36_half"]
    run_case("bf16", 1, c["hidden"], c["heads"], c["ffn"], c["micro_batch"], c["seq"], c["mem_len"], c["streams"], M=1, K=1,
             seed=c["index"], stddev=0.02, perturb=False, odtype=torch.float32, fused=True)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_forward_backward_overlap(dtype):
    # backward passes on the second stream, slots (and their masks / memories) reused three times over
    run_case(dtype, L=2, H=64, N=4, F=128, B=2, Q=16, Mm=8, S=2, M=6, seed=3, overlap=True)
