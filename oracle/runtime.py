"""CPU restatement of the reference's per-stage runtime. TEST INFRASTRUCTURE ONLY.

One stage of the unrolled graph of bert/graph.py:97-161: forward and backward
of M micro-batches in the early-backward order, a stash of at most K live
micro-batches, and the gradient accumulation of bert/graph.py:145-161
(tf.accumulate_n: a plain sum over micro-batches, no 1/M), done left to right
in the order the backward passes finish.
"""
import torch

from . import schedule


def accumulate(grads, dtype=None):
    """acc = g_0 + g_1 + ... left to right (bert/graph.py:159)."""
    acc = grads[0].clone() if dtype is None else grads[0].to(dtype).clone()
    for g in grads[1:]:
        acc += g if dtype is None else g.to(dtype)
    return acc


def run_stage(forward_fn, weights, inputs, upstream, stage=0, num_stages=2, variant="S",
              stash_limit=None):
    """Runs ``forward_fn(x, weights) -> out`` for every micro-batch under the schedule.

    Returns (outputs[M], input_grads[M] (None entries for integer inputs),
    {name: accumulated grad}, max_live) where max_live is the high-water mark of the stash."""
    M = len(inputs)
    ops = schedule.closed_form(stage, num_stages, M, variant)
    K = schedule.stash_depth(stage, num_stages, variant) if stash_limit is None else stash_limit
    names = sorted(weights)
    live = {}
    outputs, in_grads = [None] * M, [None] * M
    acc = {}
    max_live = 0
    for op, j in ops:
        if op == "F":
            x = inputs[j]
            if x.dtype.is_floating_point:
                x = x.clone().requires_grad_(True)
            out = forward_fn(x, weights)
            live[j] = (x, out)
            if len(live) > K:
                raise AssertionError("stash overflow: %d live > K=%d" % (len(live), K))
            max_live = max(max_live, len(live))
            outputs[j] = out.detach()
        else:
            x, out = live.pop(j)
            xs = ([x] if x.dtype.is_floating_point else []) + [weights[n] for n in names]
            grads = torch.autograd.grad(out, xs, grad_outputs=upstream[j], allow_unused=True)
            off = 0
            if x.dtype.is_floating_point:
                in_grads[j] = grads[0]
                off = 1
            for n, g in zip(names, grads[off:]):
                if g is None:            # bert/graph.py:118-119 drops None grads
                    continue
                if n in acc:
                    acc[n] += g
                else:
                    acc[n] = g.clone()
    return outputs, in_grads, acc, max_live
