"""Pins the schedule rule and the accumulate semantics of the runtime oracle."""
import pytest
import torch

from dapple_amd import synthetic
from oracle import bert as ob
from oracle import runtime as ort
from oracle import schedule


@pytest.mark.parametrize("S,M,variant", [(2, 8, "S"), (2, 4, "S"), (3, 7, "S"), (4, 4, "S"), (1, 3, "S"),
                                          (2, 12, "2S-1"), (3, 9, "2S-1")])
def test_simulated_graph_order_equals_closed_form(S, M, variant):
    # the event simulation of bert/graph.py:129's dependency rule yields F0..F(K-1),B0,F(K),B1,...
    order = schedule.simulate(S, M, variant)
    closed = [schedule.closed_form(i, S, M, variant) for i in range(S)]
    # The first stage - the one whose backward never arrives early - runs exactly the closed form under both rules.  Under
    # rule "S" so does every stage.  Under "2S-1" the control edges allow stage i > 0 more forwards in flight (2S-1-i) than a
    # backward-first executor ever accumulates there (its backward is ready as soon as the stage behind it is done), so
    # the simulated order of those stages runs at a smaller depth; the closed form is then the DEEPEST order the edges
    # allow, which is what the runtime sizes the stash for and issues.
    assert order[0] == closed[0]
    if variant == "S":
        assert order == closed
    # the closed forms of all stages together are one valid execution of the unrolled graph (no edge violated, no deadlock)
    assert schedule.runs_to_completion(closed, S, M, variant)
    assert schedule.runs_to_completion(order, S, M, variant)
    bad = [list(c) for c in closed]
    if M > 1 and len(bad[0]) > 2:
        k0 = min(schedule.stash_depth(0, S, variant), M)
        if k0 < M:   # one forward more than the rule allows in front of the first backward: must deadlock
            bad[0] = [("F", j) for j in range(k0 + 1)] + [op for op in closed[0][k0:] if op != ("F", k0)]
            assert not schedule.runs_to_completion(bad, S, M, variant)
    for i in range(S):
        K = min(schedule.stash_depth(i, S, variant), M)
        for ops, exact in ((closed[i], True), (order[i], variant == "S" or i == 0)):
            live, peak, seen_f, seen_b = 0, 0, set(), set()
            for op, j in ops:
                if op == "F":
                    live += 1
                    seen_f.add(j)
                else:
                    assert j in seen_f          # every F_j precedes B_j
                    live -= 1
                    seen_b.add(j)
                peak = max(peak, live)
            assert (peak == K if exact else peak <= K) and seen_f == seen_b == set(range(M))


def test_dep_rule_truth_table():
    # S=2: stage 0 waits on F(j-1) only for j=1, then on B(j-2); stage 1 always on B(j-1)
    assert schedule.dep_of(1, 0, 2) == ("F", 0)
    assert schedule.dep_of(2, 0, 2) == ("B", 0)
    assert schedule.dep_of(5, 0, 2) == ("B", 3)
    assert schedule.dep_of(1, 1, 2) == ("B", 0)
    assert schedule.dep_of(0, 1, 2) is None
    assert schedule.dep_of(2, 0, 2, "2S-1") == ("F", 1)
    assert schedule.dep_of(3, 0, 2, "2S-1") == ("B", 0)
    assert schedule.stash_depth(0, 2) == 2 and schedule.stash_depth(1, 2) == 1
    assert schedule.stash_depth(0, 2, "2S-1") == 3


def test_accumulate_is_left_to_right_fp32_sum():
    g = [torch.tensor([1e8], dtype=torch.float32), torch.tensor([1.0], dtype=torch.float32),
         torch.tensor([-1e8], dtype=torch.float32), torch.tensor([1.0], dtype=torch.float32)]
    # ((1e8 + 1) - 1e8) + 1 == 1 in fp32 (the first +1 is absorbed): order matters and is fixed
    assert ort.accumulate(g).item() == 1.0
    assert ort.accumulate(g, torch.float64).item() == 2.0


def test_accumulated_grads_equal_grad_of_concatenated_batch_and_do_not_depend_on_K():
    B, S, N, H, F, M = 1, 4, 2, 8, 16, 4
    w = ob.to_torch(synthetic.bert_weights(21, 2, H, F, stddev=0.3, perturb=True), requires_grad=True)
    xs = [torch.randn(B * S, H, dtype=torch.float64) for _ in range(M)]
    dys = [torch.randn(B * S, H, dtype=torch.float64) for _ in range(M)]
    fwd = lambda x, ww: ob.stage_forward(x, ww, [0, 1], B, S, N)
    outs, dxs, acc, peak = ort.run_stage(fwd, w, xs, dys, stage=0, num_stages=2)
    assert peak == 2
    # sum over micro-batches == gradient of one batch made of all micro-batches (no 1/M)
    big = torch.cat(xs).requires_grad_(True)
    out = ob.stage_forward(big, w, [0, 1], B * M, S, N)
    names = sorted(w)
    grads = torch.autograd.grad(out, [big] + [w[n] for n in names], torch.cat(dys))
    assert torch.allclose(torch.cat(dxs), grads[0], atol=1e-12)
    for n, g in zip(names, grads[1:]):
        assert torch.allclose(acc[n], g, atol=1e-10), n
    for K in (1, 3, 4):
        o2, dx2, acc2, _ = ort.run_stage(fwd, w, xs, dys, stage=0, num_stages=2, stash_limit=K) if K >= 2 else \
            ort.run_stage(fwd, w, xs, dys, stage=1, num_stages=2)
        for a, b in zip(outs, o2):
            assert torch.equal(a, b)
        for n in names:
            assert torch.equal(acc[n], acc2[n])


def test_stash_overflow_is_detected():
    w = ob.to_torch(synthetic.bert_weights(1, 1, 8, 16), requires_grad=True)
    xs = [torch.randn(4, 8, dtype=torch.float64) for _ in range(3)]
    fwd = lambda x, ww: ob.stage_forward(x, ww, [0], 1, 4, 2)
    with pytest.raises(AssertionError):
        ort.run_stage(fwd, w, xs, xs, stage=0, num_stages=2, stash_limit=1)
