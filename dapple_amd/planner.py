"""Stage planner: which layers go on which pipeline stage, how many replicas each stage gets.

A Python restatement of the reference's HPGO planner (Rust, with the profile graph handled by a Python script it
embeds): profile file -> antichain states (src/input/torch_graph_py.rs:301-460, 658-792) -> model normalised to
the global batch (src/model/model.rs:49-150) -> device placements (src/environment/device.rs:37-294) -> the
dynamic program over (state, pipeline slots, occupied-GPU set) (src/orchestration/orchestrate.rs:81-428) -> the
analytical speed-up of a synchronous pipeline (src/parallelism/sync_pipeline.rs:23-135) with the all-reduce and
split/concat cost models (src/parallelism/data_parallel.rs:6-16, split_concat.rs:4-39) -> the best of all plans
(orchestrate.rs:430-690).  The bandwidth constants are the reference's (25 GB/s inside a machine, 3 GB/s
collectives and 1 GB/s point-to-point between machines); pass others through ``Network`` for another fabric.

Where the reference iterates a hash map (candidate placements) the order here is the sorted order of the GPU
sets, so a run is reproducible; ties between equal plans may therefore resolve differently than in a given
run of the reference, whose own order changes from run to run.

Host-side logic only: nothing here touches the GPU.
"""
import collections

GIGABYTE = 1e9


class Network(object):
    """Bandwidths in bytes/s (src/environment/nvlink.rs, ethernet.rs)."""

    def __init__(self, intra_p2p=25.0 * GIGABYTE, inter_p2p=1.0 * GIGABYTE, inter_collective=3.0 * GIGABYTE):
        self.intra_p2p, self.inter_p2p, self.inter_collective = intra_p2p, inter_p2p, inter_collective


# ------------------------------------------------------------------------------------------- profile graph
class Node(object):
    def __init__(self, node_id, desc="", fwd=0.0, bwd=0.0, activation=0.0, parameters=0.0):
        self.node_id, self.desc = node_id, desc
        self.forward_compute_time, self.backward_compute_time = fwd, bwd
        self.activation_size, self.parameter_size = activation, parameters


def parse_node(line):
    """``node5 -- layer_0 -- forward_compute_time=2.69, backward_compute_time=4.47, activation_size=4325376,
    parameter_size=50384896``; an activation size may be a list ``[a; b]`` (summed) (torch_graph_py.rs:658-677)."""
    tok = line.strip().split(" -- ")
    meta = tok[2].split(", ")
    if len(meta) != 4:
        raise ValueError("profile node line with %d metadata fields: %r" % (len(meta), line))
    val = [m.split("=", 1)[1] for m in meta]
    act = val[2]
    if "[" in act:
        act = sum(float(x) for x in act.lstrip("[").rstrip("]").split("; "))
    return Node(tok[0], tok[1], float(val[0]), float(val[1]), float(act), float(val[3]))


class ProfileGraph(object):
    """Nodes and edges of a profile file; edges are the indented ``nodeA -- nodeB`` lines."""

    def __init__(self):
        self.nodes = collections.OrderedDict()
        self.out, self.inc = collections.defaultdict(list), collections.defaultdict(list)
        self._pred, self._succ = {}, {}

    @classmethod
    def from_str(cls, text):
        g = cls()
        for line in text.strip().split("\n"):
            if not line.strip():
                continue
            if not line.startswith((" ", "\t")):
                n = parse_node(line)
                g.nodes[n.node_id] = n
            else:
                a, b = line.strip().split(" -- ")
                g.out[a].append(b)
                g.inc[b].append(a)
        return g

    def remove(self, nid):
        del self.nodes[nid]
        for b in self.out.pop(nid, []):
            self.inc[b].remove(nid)
        for a in self.inc.pop(nid, []):
            self.out[a].remove(nid)
        self._pred, self._succ = {}, {}

    def sources(self):
        return [n for n in self.nodes if not self.inc.get(n)]

    def sinks(self):
        return [n for n in self.nodes if not self.out.get(n)]

    def _closure(self, nid, edges, memo):
        # transitive closure without recursion (profiles have a few hundred nodes in a chain)
        if nid in memo:
            return memo[nid]
        order, seen, stack = [], set(), [nid]
        while stack:
            v = stack[-1]
            todo = [u for u in edges.get(v, []) if u not in memo and u not in seen]
            if todo:
                seen.add(todo[0])
                stack.append(todo[0])
                continue
            stack.pop()
            if v in memo:
                continue
            acc = set()
            for u in edges.get(v, []):
                acc.add(u)
                acc |= memo[u]
            memo[v] = acc
            order.append(v)
        return memo[nid]

    def predecessors(self, nid):
        return self._closure(nid, self.inc, self._pred)

    def successors(self, nid):
        return self._closure(nid, self.out, self._succ)

    # -- antichains: a set of nodes no two of which are ordered = one cut of the graph
    def augment(self, antichain):
        """The antichain plus every earlier node whose output is still needed on the far side of the cut
        (it has an edge to a node that is neither before the antichain node nor that node itself)."""
        extra = []
        for a in antichain:
            before = self.predecessors(a)
            for p in before:
                if p in extra:
                    continue
                if any(o not in before and o != a for o in self.out.get(p, [])):
                    extra.append(p)
        return [p for p in self.nodes if p in extra] + list(antichain)

    def deaugment(self, nodes):
        """Drops every node that has a successor inside the set: what is left is an antichain again."""
        drop = set()
        for a in nodes:
            succ = self.successors(a)
            if any(b in succ for b in nodes):
                drop.add(a)
        out = []
        for a in nodes:
            if a not in drop and a not in out:
                out.append(a)
        return out

    def next_antichains(self, antichain):
        """Cuts one step later: one node of the augmented antichain advances along one of its edges, allowed when
        nothing after the new node is still in the set."""
        aug = self.augment(antichain)
        aug_set, cur = set(aug), set(antichain)
        res = []
        for a in aug:
            for nxt in self.out.get(a, []):
                if nxt in cur:
                    continue
                if any(s in aug_set for s in self.successors(nxt)):
                    continue
                res.append(self.deaugment([nxt if x == a else x for x in aug]))
        return res


class State(object):
    """One cut of the model: everything before it can form the leading stages."""

    def __init__(self, index, antichain, desc):
        self.index, self.antichain, self.desc = index, antichain, desc
        self.compute_time = self.activation_size = self.parameter_size = self.output_activation_size = 0.0


def antichain_states(g):
    """States in topological order of the antichain DAG and, per state, the indices of all states before it."""
    first = [g.sources()[0]]
    key = lambda a: tuple(sorted(a))
    ids = {key(first): 0}
    chains = [first]
    edges = collections.defaultdict(list)
    queue, done = [first], set()
    while queue:
        a = queue.pop(0)
        if key(a) in done:
            continue
        done.add(key(a))
        for n in g.next_antichains(a):
            if key(n) not in ids:
                ids[key(n)] = len(chains)
                chains.append(n)
            edges[ids[key(a)]].append(ids[key(n)])
            queue.append(n)
    descs = [g.nodes[c[0]].desc for c in chains]
    # depth-first topological order, roots and children taken by description (then by creation order)
    order, mark = [], set()
    for root in sorted(range(len(chains)), key=lambda i: (descs[i], i)):
        if root in mark:
            continue
        stack = [(root, iter(sorted(set(edges[root]), key=lambda i: (descs[i], i))))]
        onpath = {root}
        while stack:
            v, it = stack[-1]
            nxt = next((u for u in it if u not in mark), None)
            if nxt is None:
                stack.pop()
                onpath.discard(v)
                if v not in mark:
                    mark.add(v)
                    order.insert(0, v)
                continue
            if nxt in onpath:
                raise ValueError("profile graph has a cycle")
            onpath.add(nxt)
            stack.append((nxt, iter(sorted(set(edges[nxt]), key=lambda i: (descs[i], i)))))
    pos = {v: i for i, v in enumerate(order)}
    inc = collections.defaultdict(set)
    for a, outs in edges.items():
        for b in outs:
            inc[b].add(a)
    before = {}

    def all_before(v):
        if v not in before:
            acc = set()
            for u in inc[v]:
                acc.add(u)
                acc |= all_before(u)
            before[v] = acc
        return before[v]

    states, preds = [], []
    for i, v in enumerate(order):
        states.append(State(i, g.augment(chains[v]), descs[v]))
        preds.append(sorted(pos[u] for u in all_before(v)))
    return states, preds


class ModelPerf(object):
    """compute_times[0][j] = time of states 0..j; compute_times[i][j] (i >= 1) = time of states i..j, -1 where
    j < i.  Same for activation and parameter sizes (torch_graph_py.rs:766-792)."""

    def __init__(self, states, preds):
        self.states, self.all_predecessor_ids = states, preds
        n = len(states)

        def matrix(attr):
            v = [getattr(s, attr) for s in states]
            rows = [list(v)]
            for i in range(1, n + 1):
                rows.append([v[j] - v[i - 1] if j > i - 1 else -1.0 for j in range(n)])
            return rows
        self.compute_times = matrix("compute_time")
        self.activation_sizes = matrix("activation_size")
        self.parameter_sizes = matrix("parameter_size")
        self.output_activation_sizes = [s.output_activation_size for s in states]


def prepare(profile_text):
    """Profile text -> ModelPerf (torch_graph_py.rs:695-792): ``Input*`` sources and ``__getitem__`` sinks are dropped,
    every state gets the summed forward + backward time (ms -> s), activation and parameter bytes of everything
    before its cut, and the bytes that cross the cut."""
    g = ProfileGraph.from_str(profile_text)
    for s in g.sources():
        if g.nodes[s].desc.startswith("Input"):
            g.remove(s)
    for s in g.sinks():
        if g.nodes[s].desc.startswith("__getitem__"):
            g.remove(s)
    states, preds = antichain_states(g)
    for st in states:
        st.output_activation_size = sum(g.nodes[a].activation_size for a in st.antichain)
        members = set()
        for a in st.antichain:
            members |= g.predecessors(a)
            members.add(a)
        for nid in members:
            n = g.nodes[nid]
            st.compute_time += (n.forward_compute_time + n.backward_compute_time) / 1000.0
            st.activation_size += n.activation_size
            st.parameter_size += n.parameter_size
    return ModelPerf(states, preds)


class Model(object):
    """Profile normalised from the profiling batch size to the global batch size: times and activations scale,
    parameters do not (src/model/model.rs:49-150)."""

    def __init__(self, perf, profile_batch_size, global_batch_size):
        self.perf = perf
        self.profile_batch_size, self.global_batch_size = profile_batch_size, global_batch_size
        self.min_micro_batch_size = 1
        self.optimizer_memory_scaling = 1
        self.peak_activation_per_batch = perf.activation_sizes[0][-1] / float(profile_batch_size)
        f = float(global_batch_size) / float(profile_batch_size)
        perf.compute_times = [[c * f for c in row] for row in perf.compute_times]
        perf.activation_sizes = [[c * f for c in row] for row in perf.activation_sizes]
        perf.output_activation_sizes = [c * f for c in perf.output_activation_sizes]
        n = len(perf.compute_times[0])
        self.layers = [dict(id=i, desc=perf.states[i].desc, compute_time=perf.compute_times[i][i],
                            activation_size=perf.activation_sizes[i][i],
                            output_activation_size=perf.output_activation_sizes[i],
                            parameter_size=perf.parameter_sizes[i][i]) for i in range(n)]


# ------------------------------------------------------------------------------------------- devices
Placement = collections.namedtuple("Placement", "strategy occupied gids")


class Devices(object):
    """``n`` GPUs; ``seps`` = the running GPU count at the end of every machine, e.g. [8, 16]
    (src/environment/device.rs:37-48)."""

    def __init__(self, n, seps, network=None):
        self.num_gpus, self.seps, self.num_machines = n, list(seps), len(seps)
        self.network = network or Network()
        self._replica_memo = {}

    def _one_machine(self, lo, hi):
        l = 0
        for r in self.seps:
            if l <= lo < r and l <= hi < r:
                return True
            l = r
        return False

    def is_cross_machine_within(self, gids):
        return not self._one_machine(min(gids), max(gids))

    def is_cross_machine_from_to(self, a, b):
        return not self._one_machine(min(min(a), min(b)), max(max(a), max(b)))

    def _with_strategy(self, occupied, need, avail, strategy):
        occ, gids, left = list(occupied), set(), need
        avail = [list(a) for a in avail]
        start = lambda i: 0 if i == 0 else self.seps[i - 1]
        if strategy == "scatter":
            while left > 0:
                progressed = False
                for i in range(len(avail)):
                    if avail[i][1] > 0 and left > 0:
                        j = start(i)
                        while occ[j]:
                            j += 1
                        occ[j] = True
                        gids.add(j)
                        left -= 1
                        avail[i][1] -= 1
                        progressed = True
                if not progressed:
                    break
        else:
            fresh = strategy == "fresh"
            for i in range(len(avail)):
                if avail[i][0] != fresh:
                    continue
                j = start(i)
                if avail[i][1] >= left:
                    while occ[j] and j < len(occ) - 1:
                        j += 1
                    while left > 0:
                        occ[j] = True
                        gids.add(j)
                        j += 1
                        left -= 1
                else:
                    while j < len(occ) and occ[j]:     # (the reference indexes past the end here when nothing later is free)
                        j += 1
                    while j < self.seps[i]:
                        occ[j] = True
                        gids.add(j)
                        j += 1
                        left -= 1
        return Placement(strategy, tuple(occ), frozenset(gids)) if left == 0 else None

    def next_cards(self, occupied, need):
        """Candidate placements of ``need`` more GPUs: whole fresh machines first, partly used machines first, or
        one per machine in turn; duplicates (same GPU set) collapse (device.rs:182-229)."""
        avail, lo, total = [], 0, 0
        for s in self.seps:
            free = sum(1 for i in range(lo, s) if not occupied[i])
            avail.append((free == s - lo, free))
            total += free
            lo = s
        if total < need:
            raise ValueError("next_cards: %d GPUs needed, %d free" % (need, total))
        found = {}
        for strategy in ("fresh", "append", "scatter"):
            r = self._with_strategy(occupied, need, avail, strategy)
            if r is not None:
                found[r.gids] = r
        return [found[k] for k in sorted(found, key=sorted)]

    def next_cards_with_replica(self, occupied, need, replica):
        """``replica`` rounds of ``need`` GPUs, every combination of the rounds' strategies, merged per resulting
        GPU set (device.rs:231-293)."""
        memo_key = (tuple(occupied), need, replica)
        if memo_key in self._replica_memo:          # the search asks for the same placement for every pair of cuts
            return self._replica_memo[memo_key]
        rounds = [([], tuple(occupied))]
        for _ in range(replica):
            nxt = []
            for gids, occ in rounds:
                for p in self.next_cards(occ, need):
                    nxt.append((gids + sorted(p.gids), p.occupied))
            rounds = nxt
        found = {}
        for gids, occ in rounds:
            found[frozenset(gids)] = Placement("fusion", occ, frozenset(gids))
        self._replica_memo[memo_key] = [found[k] for k in sorted(found, key=sorted)]
        return self._replica_memo[memo_key]

    # -- cost models
    def all_reduce_time(self, gids, size):
        n = len(gids)
        if n == 1:
            return 0.0
        f = (n - 1) / float(n)
        if self.is_cross_machine_within(gids):
            return size * 2.0 * f / self.network.inter_collective
        return size * 2.0 * f / self.network.intra_p2p / float(n // 2)

    def split_concat_all2all_time(self, src, dst, size):
        if not self.is_cross_machine_within(dst):
            cross = [s for s in src if self.is_cross_machine_from_to([s], dst)]
            if cross:
                return size / float(len(src)) * len(cross) / self.network.inter_p2p
            return size / self.network.intra_p2p
        if self.is_cross_machine_from_to(src, dst):
            return size / self.network.inter_collective
        return size / self.network.intra_p2p


# ------------------------------------------------------------------------------------------- the plan
Cell = collections.namedtuple("Cell", "block split num_used came_from gids")
Plan = collections.namedtuple("Plan", "speedup stages replicas")     # stages: (first state, end, slots, GPU ids)
_BEST = "best"                                                        # the key the reference keeps as an all-true bitset


def sync_pipeline_speedup_analytical(d, m, rp, pipeline_time, stages):
    """Speed-up over one GPU of a synchronous pipeline (sync_pipeline.rs:23-135): the bottleneck block repeated for
    every micro-batch but one, one pass of the whole model at micro-batch size, the boundary transfers, and whatever
    of the stages' gradient all-reduces the earlier stages' drain does not hide."""
    perf = m.perf
    total = perf.compute_times[0][-1]
    m_batch = m.global_batch_size // rp // m.min_micro_batch_size
    if m_batch == 0:
        return 0.0
    block = pipeline_time / m_batch
    length = block * (m_batch - 1) + total / rp / m_batch
    for i in range(len(stages) - 1):
        cut = perf.output_activation_sizes[stages[i][1] - 1] / rp / m_batch
        length += d.split_concat_all2all_time(stages[i][3], stages[i + 1][3], cut)
    delta = 0.0
    for i, s in enumerate(stages):
        ar = d.all_reduce_time(s[3], perf.parameter_sizes[s[0]][s[1]])
        if ar > i * block:
            delta = max(ar - i * block, delta)
    return total / (length + delta)


class SyncOrchestrate(object):
    """``SyncOrchestrate(profile text, profile batch size, global batch size, seps)`` then ``orchestrate()``: the
    reference's ``conductor_from_torch_graph_and_seps(...).py_orchestrate()`` (orchestrate.rs:52-70, 614-631)."""

    def __init__(self, profile_text, pbs, gbs, seps, network=None, min_micro_batch_size=1):
        self.m = Model(prepare(profile_text), pbs, gbs)
        self.m.min_micro_batch_size = min_micro_batch_size
        self.d = Devices(seps[-1], seps, network)
        self.res = []

    @classmethod
    def from_file(cls, path, pbs, gbs, seps, **kw):
        with open(path) as f:
            return cls(f.read(), pbs, gbs, seps, **kw)

    def compute_plan_sync(self, slots, rp, straight):
        """A[j][m][occupied GPUs] = the smallest bottleneck (longest stage or transfer) of states 0..j on m + 1
        pipeline slots of ``rp`` replicas each, ending in that GPU occupancy (orchestrate.rs:81-378)."""
        perf, d = self.m.perf, self.d
        ct, oas, preds = perf.compute_times, perf.output_activation_sizes, perf.all_predecessor_ids
        n = len(ct[0])
        A = [[dict() for _ in range(slots)] for _ in range(n)]
        empty = tuple([False] * d.num_gpus)
        for j in range(n):
            for m in range(1 if straight else slots):
                cands = d.next_cards(empty, (m + 1) * rp)
                first = next((c for c in cands if c.strategy == "fresh"), cands[0])
                cell = Cell(max(ct[0][j] / (m + 1) / rp, 0.0), None, m + 1, empty, first.gids)
                A[j][m][_BEST] = cell
                A[j][m][first.occupied] = cell
        skip_real = d.num_gpus > slots * rp       # the reference's test for its marker key also drops real keys then
        for m in range(1, slots):
            for j in range(1, n):
                cur = A[j][m]
                best = cur.get(_BEST, Cell(None, None, None, (), frozenset()))
                for k in preds[j]:
                    for mp in range(1, 2 if straight else m + 1):
                        prev = A[k][m - mp]
                        if _BEST not in prev or prev[_BEST].block is None:
                            continue
                        stage_time = ct[k + 1][j]
                        if stage_time < -0.5:
                            continue
                        stage_time /= float(mp * rp)
                        for occ in sorted(key for key in prev if key != _BEST):
                            if skip_real:
                                continue
                            cell = prev[occ]
                            for nb in d.next_cards_with_replica(occ, mp, rp):
                                transfer = d.split_concat_all2all_time(cell.gids, nb.gids, 2.0 * oas[k])
                                t = max(cell.block, stage_time, transfer)
                                if best.block is None or t < best.block:
                                    best = Cell(t, (k, m - mp), mp, occ, nb.gids)
                                if nb.occupied not in cur or t < cur[nb.occupied].block:
                                    cur[nb.occupied] = Cell(t, (k, m - mp), mp, occ, nb.gids)
                cur[_BEST] = best
        return A

    def analyse_plan_sync(self, A, end, slots):
        """Walks the optimal splits back from the last state (orchestrate.rs:381-428).  A stage is (first state,
        end, slots used, GPU ids); ``end`` is one past the stage's last state except for the last stage, where it
        is the last state itself - the reference's convention, kept because the speed-up model indexes with it."""
        res = []
        meta = A[end - 1][slots - 1][_BEST]
        if not meta.gids:
            raise RuntimeError("no plan: the last stage has no GPUs")
        prev_split = end - 1
        while meta.split is not None:
            res.append((meta.split[0] + 1, prev_split, meta.num_used, meta.gids))
            prev_split = res[-1][0]
            meta = A[meta.split[0]][meta.split[1]][meta.came_from]
        res.append((0, prev_split, meta.num_used, meta.gids))
        res.reverse()
        return res

    def plan_for(self, slots, straight):
        rp = self.d.num_gpus // slots
        A = self.compute_plan_sync(slots, rp, straight)
        n = len(self.m.perf.compute_times[0])
        t = A[n - 1][slots - 1][_BEST].block
        if t is None or t < 0.001:
            raise RuntimeError("pipeline time error")
        stages = self.analyse_plan_sync(A, n, slots)
        return Plan(sync_pipeline_speedup_analytical(self.d, self.m, rp, t, stages), stages, rp)

    def compute_bipartition(self):
        """Every two-stage plan: cut after any state, g GPUs before the cut and the rest after it, every placement
        (orchestrate.rs:430-531)."""
        perf, d = self.m.perf, self.d
        ct, n = perf.compute_times, len(perf.compute_times[0])
        empty = tuple([False] * d.num_gpus)
        best = None
        for l in range(n - 1):
            for g in range(1, d.num_gpus):
                for g1 in d.next_cards(empty, g):
                    for g2 in d.next_cards(g1.occupied, d.num_gpus - g):
                        comp = max(ct[0][l] / len(g1.gids), ct[l + 1][n - 1] / len(g2.gids))
                        comm = d.split_concat_all2all_time(g1.gids, g2.gids, perf.output_activation_sizes[l])
                        stages = [(0, l + 1, len(g1.gids), g1.gids), (l + 1, n - 1, len(g2.gids), g2.gids)]
                        s = sync_pipeline_speedup_analytical(d, self.m, 1, max(comp, comm), stages)
                        if best is None or s > best.speedup:
                            best = Plan(s, stages, 1)
        return best

    def orchestrate(self):
        """All candidate plans (orchestrate.rs:647-675): every slot count 2..num_gpus, the straight pipelines, the
        bipartitions.  Returns the best as ``(speedup, [(first, end, slots, sorted GPU ids), ...])``."""
        g = self.d.num_gpus
        self.res = [self.plan_for(i, False) for i in range(2, g + 1)]
        for i in ([2, g] if g > 2 and g % 2 == 0 else [g]):
            self.res.append(self.plan_for(i, True))
        self.res.append(self.compute_bipartition())
        best = max(self.res, key=lambda r: r.speedup)
        return best.speedup, [(s[0], s[1], s[2], sorted(s[3])) for s in best.stages]


def conductor_from_torch_graph_and_seps(profile_filename, profile_batch_size, global_batch_size, seps):
    """The reference's Python entry point (src/api/pylib.rs; PLANNER_REPRODUCTION.md)."""
    return SyncOrchestrate.from_file(profile_filename, profile_batch_size, global_batch_size, seps)


def stage_layers(plan_stages, perf):
    """Descriptions of the states each stage of a plan covers, for mapping a plan onto a model's layers."""
    out = []
    for i, s in enumerate(plan_stages):
        last = s[1] if i == len(plan_stages) - 1 else s[1] - 1
        out.append([perf.states[j].desc for j in range(s[0], last + 1)])
    return out


def encoder_layer_ranges(plan_stages, perf):
    """(first layer, number of layers) of every stage, from the states named ``layer_<n>`` / ``Layer_<n>`` it covers
    (BERT and XLNet profiles): the ``first_layer`` / ``num_layers`` a stage of ``runtime.bert_stage`` or
    ``runtime.xlnet_stage`` is built with.  A stage without such states gets (None, 0)."""
    import re
    out = []
    for names in stage_layers(plan_stages, perf):
        ids = sorted(int(m.group(1)) for m in (re.match(r"^[Ll]ayer_(\d+)$", n) for n in names) if m)
        out.append((ids[0], len(ids)) if ids else (None, 0))
    return out


def micro_batches(plan, model):
    """Micro-batches per step and replica of a plan: global batch / replicas / the micro-batch size
    (sync_pipeline.rs:39, the count the speed-up model is evaluated with)."""
    return model.global_batch_size // plan.replicas // model.min_micro_batch_size

