"""CPU restatement of the reference's pipeline unroll rule. TEST INFRASTRUCTURE ONLY.

bert/graph.py:126-132 of the reference builds, for micro-batch j and stage i,
the control dependency

    dep_outputs[i] = all_outputs[j-1][i]            if i + j < S
                   = layer_grads[i + j - S][i]      otherwise

i.e. stage i may start forward j only after forward j-1 (warm-up) or after the
backward of micro-batch j-(S-i).  vgg19/tf-keras-dapple.py:292 and
amoeba_net/amoeba_net_slice_model.py:427 use ``i + j < 2S - 1`` instead.

This module states that rule as an event simulation over the whole S-stage
pipeline (every stage executes what is ready, backward first), and returns the
order one stage runs its ops in.  The closed form F0..F(K-1), B0, F(K), B1, ...
is what the tests pin it against.
"""


def dep_of(j, i, num_stages, variant="S"):
    """What forward(j) at stage i waits for: ('F', j-1) or ('B', j-K); None for j == 0."""
    if j == 0:
        return None
    bound = num_stages if variant == "S" else 2 * num_stages - 1
    if i + j < bound:
        return ("F", j - 1)
    return ("B", i + j - bound)


def stash_depth(stage, num_stages, variant="S"):
    """In-flight micro-batches at ``stage``: S - i, or 2S - 1 - i for the VGG/AmoebaNet rule."""
    return (num_stages if variant == "S" else 2 * num_stages - 1) - stage


def simulate(num_stages, num_micro_batches, variant="S"):
    """Event simulation of the unrolled graph; returns per-stage op lists [('F'|'B', j), ...].

    Edges: F(j,i) needs F(j,i-1) [data], dep_of(j,i) [control];
           B(j,i) needs F(j,i) and B(j,i+1) [data] (last stage: its own F).
    Each stage is one device running one op at a time; a ready backward wins over a
    ready forward (early backward), ties go to the smaller micro-batch."""
    S, M = num_stages, num_micro_batches
    done = set()
    order = [[] for _ in range(S)]
    total = 2 * S * M
    while len(done) < total:
        progressed = False
        fired = []
        for i in range(S):
            cand = None
            for j in range(M):
                if ("B", j, i) in done or ("F", j, i) not in done:
                    continue
                if i == S - 1 or ("B", j, i + 1) in done:
                    cand = ("B", j, i)
                    break
            if cand is None:
                for j in range(M):
                    if ("F", j, i) in done:
                        continue
                    if i > 0 and ("F", j, i - 1) not in done:
                        break
                    dep = dep_of(j, i, S, variant)
                    if dep is not None and (dep[0], dep[1], i) not in done:
                        break
                    cand = ("F", j, i)
                    break
            if cand is not None:
                fired.append(cand)
        for op in fired:
            done.add(op)
            order[op[2]].append((op[0], op[1]))
            progressed = True
        if not progressed:
            raise RuntimeError("schedule deadlock")
    return order


def closed_form(stage, num_stages, num_micro_batches, variant="S"):
    """F0..F(K-1), B0, F(K), B1, ..., F(M-1), B(M-K), ..., B(M-1) with K = stash_depth."""
    M = num_micro_batches
    K = min(stash_depth(stage, num_stages, variant), M)
    ops = [("F", j) for j in range(K)]
    for j in range(M):
        ops.append(("B", j))
        if j + K < M:
            ops.append(("F", j + K))
    return ops


def runs_to_completion(orders, num_stages, num_micro_batches, variant="S"):
    """True if every stage can execute exactly its prescribed op list ``orders[i]``, in that order, without deadlock
    under the graph's edges (the data edges of ``simulate`` and the control edge ``dep_of``): the prescribed lists are
    then one valid execution of the reference's unrolled graph."""
    S = num_stages
    pos = [0] * S
    done = set()
    total = sum(len(o) for o in orders)
    while len(done) < total:
        fired = []
        for i in range(S):
            if pos[i] >= len(orders[i]):
                continue
            op, j = orders[i][pos[i]]
            if op == "F":
                ok = (i == 0 or ("F", j, i - 1) in done)
                dep = dep_of(j, i, S, variant)
                ok = ok and (dep is None or (dep[0], dep[1], i) in done)
            else:
                ok = ("F", j, i) in done and (i == S - 1 or ("B", j, i + 1) in done)
            if ok:
                fired.append((op, j, i))
        if not fired:
            return False
        for op, j, i in fired:
            done.add((op, j, i))
            pos[i] += 1
    return True
