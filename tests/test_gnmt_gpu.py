"""GNMT encoder stage parity through the C ABI against the fp64 CPU oracle (fp32: 1e-4 relative)."""
import numpy as np
import pytest
import torch

from dapple_amd import runtime, synthetic
from oracle import gnmt as og
from util import assert_close, dev

pytestmark = pytest.mark.gpu
TOL = 1e-4


def run_case(L, U, V, B, T, M, K=2, seed=0, init=0.1, perturb=True, odtype=torch.float64, M_check=None, lengths=None):
    w_np = synthetic.gnmt_weights(synthetic.SEED_WEIGHT + seed, L, U, V, init_weight=init, perturb=perturb)
    ids_np = synthetic.gnmt_id_inputs(synthetic.SEED_INPUT + seed, M, B, T, V)
    dys_np = synthetic.upstream_grads(synthetic.SEED_GRAD + seed, M, (T, B, U))
    stage = runtime.gnmt_stage(L, U, V, B, T, stash_slots=K)
    assert stage.weight_names == [synthetic.GNMT_SCOPE + "embedding_encoder"] + \
        [s + sfx for s in synthetic.gnmt_cell_scopes(L) for sfx in ("/kernel", "/bias")]
    stage.bind(w_np)
    ids, dys = [dev(i) for i in ids_np], [dev(d) for d in dys_np]
    outs = [torch.empty(T, B, U, device="cuda") for _ in range(M)]
    lens = None if lengths is None else [torch.tensor(l, dtype=torch.int32, device="cuda") for l in lengths]
    before = None if lens is None else (lambda slot, j: stage.set_lengths(slot, lens[j]))
    runtime.StageRuntime(stage, 0, K, M).step(ids, dys, outs, before_forward=before)
    stage.sync()
    w_t = og.to_torch(w_np, odtype, requires_grad=True)
    acc = {}
    for j in range(M):
        out, _, dw = og.stage_vjp(ids[j].cpu(), w_t, dys[j].cpu().to(odtype), L,
                                  lengths=None if lengths is None else torch.tensor(lengths[j]))
        if lengths is not None:
            for b, n in enumerate(lengths[j]):
                assert float(outs[j][n:, b].abs().max() if n < T else 0.0) == 0.0   # zeros past the end, exactly
        assert_close(outs[j], out, TOL, "output mb%d" % j)
        for n, g in dw.items():
            acc[n] = g.clone() if n not in acc else acc[n] + g
    for n in stage.weight_names:
        assert_close(stage.grads[n], acc[n], TOL, "accumulated grad " + n)
    stage.close()


def test_small_four_layers():
    run_case(L=4, U=32, V=50, B=4, T=6, M=3, init=0.4)


def test_two_layers_no_residual_single_step_sequence():
    run_case(L=2, U=16, V=20, B=4, T=1, M=2, K=1, seed=1, init=0.5)


def test_repeated_ids_accumulate_in_the_embedding_gradient():
    run_case(L=3, U=16, V=3, B=8, T=5, M=2, seed=2, init=0.5)


def test_config2_shape_reduced_depth():
    # BASELINE configs[2] at its real cell shape (units 1024, batch 64, seq 50, vocab 32000): the
    # bidirectional layer, uni layer 1 (2048 -> 1024) and one residual layer; one micro-batch
    c = synthetic.CONFIGS["gnmt16_encoder"]
    run_case(L=3, U=c["units"], V=c["vocab"], B=c["micro_batch"], T=c["seq"], M=1, K=1, seed=c["index"], perturb=False)


def test_ragged_sequences():
    """source_sequence_length per micro-batch: full, single-step, empty and in-between sequences; the second
    micro-batch reuses a slot whose previous lengths were different, the third goes back to full length."""
    run_case(L=4, U=32, V=50, B=4, T=6, M=3, init=0.4, seed=3, lengths=[[6, 1, 3, 5], [2, 6, 0, 4], [6, 6, 6, 6]])
