"""Small fixed launches for hardware-counter runs.

``accumulate N``: ``ds_grad_accumulate`` over N fp32 elements - known traffic (reads 8*N bytes, writes
4*N bytes), used to scale the FETCH_SIZE / WRITE_SIZE counters.
``gemms``: the GEMMs of one BERT-48 half-stage layer at their real shapes (2x512 rows, hidden 1024,
ffn 4096, bf16), three launches each in the order of the list in ``gemms``, so a counter run can report HBM traffic per launch.

``elementwise``: the HBM-bound kernels of the path at the BERT-48 half-stage's shapes, five launches each with their
algorithmic bytes printed, so a kernel trace gives achieved GB/s against the HBM peak.

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d out -o c -- python3 bench_calib.py accumulate 67108864
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d out -o g -- python3 bench_calib.py gemms
    rocprofv3 --kernel-trace --stats -d out -o e -- python3 bench_calib.py elementwise

``gemm_table``: the same GEMMs (and 4096 x 4096 x 4096) timed with events, 50 launches back to back on one stream, this
library beside ``torch.matmul`` (hipBLASLt / rocBLAS) on the same operands: TFLOP/s per shape.

``attention``: the fused attention kernels at the BERT-48 half-stage's shape (2 samples, 16 heads, 512 positions, head
size 64, bf16), three launches each, for the same counter runs as ``gemms`` (matrix-core busy cycles, HBM traffic).

``xl_scores``: the score kernels of XLNet's relative attention at the XLNet-36 half-stage's shape (two streams of 512
positions + 384 memory positions, 16 heads, head size 64, bf16, masks and segments), five launches each, with their
algorithmic bytes and FLOP printed.

``grouped``: pairs and triples of the layer's GEMMs that a stage in steady state holds at the same time (a forward product
of micro-batch j+1, an input-gradient product of micro-batch j, a weight-gradient product over four micro-batches), timed
three ways - back to back on one stream, side by side on two / three streams, and as ONE ``ds_gemm_grouped`` launch per
tile-shape choice.

``timeline [workload]``: where a step of ``bench.py``'s workload (default bert48_half) spends its time - the moment every
backward pass's chain of kernels ends (an event on a probe stream behind ``ds_stage_wait_backward``), the distance from
one to the next and what is left after the last; three steps, no profiler.
"""
import time
import sys

import torch

from dapple_amd import ops
from dapple_amd._lib import DS_EPI_ACCUM, DS_K_MAJOR, DS_MN_MAJOR


def accumulate(n):
    acc = torch.zeros(n, device="cuda")
    g = torch.ones(n, device="cuda")
    for _ in range(3):
        ops.grad_accumulate(acc, g)
    torch.cuda.synchronize()
    print("accumulate_kernel<float>: %d elements, reads %d bytes, writes %d bytes per launch" % (n, 8 * n, 4 * n))


def layer_shapes():
    rows, h, f = 1024, 1024, 4096
    return [  # name, m, n, k, a_major, b_major, accumulate
        ("fwd ffn1", rows, f, h, DS_K_MAJOR, DS_MN_MAJOR, False),
        ("fwd ffn2", rows, h, f, DS_K_MAJOR, DS_MN_MAJOR, False),
        ("dgrad ffn2", rows, f, h, DS_K_MAJOR, DS_K_MAJOR, False),
        ("wgrad ffn1", h, f, rows, DS_MN_MAJOR, DS_MN_MAJOR, True),
        ("dgrad ffn1", rows, h, f, DS_K_MAJOR, DS_K_MAJOR, False),
        ("dgrad qkv", rows, h, 3 * h, DS_K_MAJOR, DS_K_MAJOR, False),
        ("dgrad ao", rows, h, h, DS_K_MAJOR, DS_K_MAJOR, False),
        ("wgrad ffn1 x4", h, f, 4 * rows, DS_MN_MAJOR, DS_MN_MAJOR, True),   # four micro-batches in one GEMM
        ("fwd qkv", rows, 3 * h, h, DS_K_MAJOR, DS_MN_MAJOR, False),
        ("fwd ao", rows, h, h, DS_K_MAJOR, DS_MN_MAJOR, False),
        ("square 4096", 4096, 4096, 4096, DS_K_MAJOR, DS_MN_MAJOR, False),
    ]


def gemms():
    bf = torch.bfloat16
    for name, m, n, k, am, bm, acc in layer_shapes():
        a = torch.randn((m, k) if am == DS_K_MAJOR else (k, m), device="cuda").to(bf)
        b = torch.randn((n, k) if bm == DS_K_MAJOR else (k, n), device="cuda").to(bf)
        c = torch.zeros(m, n, device="cuda", dtype=torch.float32 if acc else bf)
        for _ in range(3):
            ops.gemm(a, b, c, m, n, k, am, bm, flags=DS_EPI_ACCUM if acc else 0)
        torch.cuda.synchronize()
        alg = 2 * (m * k + n * k) + (8 if acc else 2) * m * n
        print("%s: m=%d n=%d k=%d, algorithmic bytes %d" % (name, m, n, k, alg))


def gemm_table():
    bf = torch.bfloat16
    reps = 50
    print("%-16s %-22s %10s %10s %12s %12s" % ("shape", "m x n x k", "ours us", "torch us", "ours TFLOP/s", "torch TFLOP/s"))
    for name, m, n, k, am, bm, acc in layer_shapes():
        a = torch.randn((m, k) if am == DS_K_MAJOR else (k, m), device="cuda").to(bf)
        b = torch.randn((n, k) if bm == DS_K_MAJOR else (k, n), device="cuda").to(bf)
        c = torch.zeros(m, n, device="cuda", dtype=torch.float32 if acc else bf)
        ta = a if am == DS_K_MAJOR else a.t()      # [m, k] view
        tb = b.t() if bm == DS_K_MAJOR else b      # [k, n] view
        tc = torch.zeros(m, n, device="cuda", dtype=bf)

        def ours():
            ops.gemm(a, b, c, m, n, k, am, bm, flags=DS_EPI_ACCUM if acc else 0)

        def theirs():
            # the accumulating product has no single torch call on bf16 operands with an fp32 C: timed as the product alone
            torch.matmul(ta, tb, out=tc)
        us = []
        for fn in (ours, theirs):
            for _ in range(5):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            us.append(e0.elapsed_time(e1) * 1e3 / reps)
        fl = 2.0 * m * n * k
        print("%-16s %-22s %10.2f %10.2f %12.1f %12.1f" % (name + (" C+=" if acc else ""), "%d x %d x %d" % (m, n, k), us[0], us[1],
                                                          fl / us[0] / 1e6, fl / us[1] / 1e6), flush=True)


def grouped():
    bf = torch.bfloat16
    shapes = {name: (m, n, k, am, bm, acc) for name, m, n, k, am, bm, acc in layer_shapes()}
    sets = [
        ("fwd ffn1", "dgrad ffn2"),
        ("fwd qkv", "dgrad ffn2"),
        ("fwd ffn2", "dgrad ffn1"),
        ("fwd ffn2", "dgrad qkv"),
        ("fwd ao", "dgrad ao"),
        ("fwd ffn1", "dgrad ffn2", "wgrad ffn1 x4"),
        ("fwd ffn2", "dgrad ffn1", "wgrad ffn1 x4"),
        ("fwd ao", "dgrad ao", "wgrad ffn1 x4"),
        ("wgrad ffn1 x4",),
        ("fwd ffn1",),
        ("fwd ffn2",),
    ]
    reps = 20
    streams = [torch.cuda.Stream() for _ in range(3)]
    main = torch.cuda.Stream()

    def operands(name):
        m, n, k, am, bm, acc = shapes[name]
        a = torch.randn((m, k) if am == DS_K_MAJOR else (k, m), device="cuda").to(bf)
        b = torch.randn((n, k) if bm == DS_K_MAJOR else (k, n), device="cuda").to(bf)
        c = torch.zeros(m, n, device="cuda", dtype=torch.float32 if acc else bf)
        return dict(a=a, b=b, c=c, m=m, n=n, k=k, a_major=am, b_major=bm, flags=DS_EPI_ACCUM if acc else 0)

    def timed(fn):
        """`reps` rounds of fn captured into a graph (so that the host's issue rate is out of the picture), replayed."""
        with torch.cuda.stream(main):
            fn()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=main):
                for _ in range(reps):
                    fn()
            graph.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(3):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (3 * reps)

    print("%-44s %9s %9s | grouped launch, us (tile shape per problem: 0=256x256 1=256x128 2=128x128 3=128x64, 4/5 = 2/3 with two "
          "tile buffers)" % ("set", "1 stream", "n streams"))
    for names in sets:
        probs = [operands(nm) for nm in names]
        flop = sum(2.0 * p["m"] * p["n"] * p["k"] for p in probs)

        def serial():
            for p in probs:
                ops.gemm(**p)

        def side_by_side():
            cur = torch.cuda.current_stream()
            for p, st in zip(probs[1:], streams):
                st.wait_stream(cur)
                with torch.cuda.stream(st):
                    ops.gemm(**p)
            ops.gemm(**probs[0])
            for p, st in zip(probs[1:], streams):
                cur.wait_stream(st)

        t1 = timed(serial)
        tn = timed(side_by_side) if len(probs) > 1 else float("nan")
        cells = []
        narrow = [p["n"] == 1024 and p["m"] == 1024 for p in probs]
        choices = set()
        for wide_cfg in (1, 2, 4):
            for narrow_cfg in (2, 3, 4, 5):
                for wg_cfg in (0, 1, 2, 4):
                    choices.add(tuple((wg_cfg if p["flags"] else (narrow_cfg if nr else wide_cfg)) for p, nr in zip(probs, narrow)))
        for cfgs in sorted(choices):
            plist = [dict(p, cfg=c) for p, c in zip(probs, cfgs)]
            cells.append("%s:%.1f" % ("".join(str(c) for c in cfgs), timed(lambda: ops.gemm_grouped(plist))))
        print("%-44s %9.1f %9.1f | %s   [%.1f GFLOP]" % (" + ".join(names), t1, tn, "  ".join(cells), flop / 1e9), flush=True)


def wgrad_group():
    """The weight-gradient products of two BERT-48 layers over all 8 micro-batches of a step (8192 rows) as ONE grouped launch
    of 256 x 128 tiles - what the stage queues twelve times per step - three launches, for counter and trace runs."""
    bf = torch.bfloat16
    rows, h, f = 8 * 1024, 1024, 4096
    probs, flop = [], 0
    for layer in range(2):
        x, ctx, a1, hh = (torch.randn(rows, w, device="cuda").to(bf) for w in (h, h, h, f))
        dz2, du, dz1, dqkv = (torch.randn(rows, w, device="cuda").to(bf) for w in (h, f, h, 3 * h))
        for a, b, m, n, extra in ((hh, dz2, f, h, {}), (a1, du, h, f, {}), (ctx, dz1, h, h, {}),
                                  (x, dqkv, h, h, dict(ldb=3 * h, batch=3, batch_inner=3, b_strides=(0, h), c_strides=(0, h * h)))):
            nb = extra.get("batch", 1)
            c = torch.zeros(nb * m, n, device="cuda")
            probs.append(dict(a=a, b=b, c=c, m=m, n=n, k=rows, a_major=DS_MN_MAJOR, b_major=DS_MN_MAJOR, flags=DS_EPI_ACCUM, cfg=1, **extra))
            flop += 2 * m * n * rows * nb
    for _ in range(3):
        ops.gemm_grouped(probs)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        ops.gemm_grouped(probs)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / 5
    print("grouped weight gradients of two layers over 8192 rows: %d tasks, %.2f GFLOP per launch, %.1f us, %.0f TFLOP/s"
          % (len(probs), flop / 1e9, dt * 1e6, flop / dt / 1e12))


def attention():
    batch, heads, seq, d = 2, 16, 512, 64
    bf = torch.bfloat16
    qkv = torch.randn(batch * seq, 3 * heads * d, device="cuda").to(bf)
    dctx = torch.randn(batch * seq, heads * d, device="cuda").to(bf)
    for _ in range(3):
        ctx, lse = ops.attention_fwd(qkv, batch, heads, seq, 0.125)
        ops.attention_bwd(qkv, ctx, lse, dctx, batch, heads, seq, 0.125)
    torch.cuda.synchronize()
    unit = batch * heads * seq * seq * d
    print("attn_fwd_kernel: %d FLOP per launch; attn_bwd_dq_kernel: %d; attn_bwd_dkv_kernel: %d" % (4 * unit, 6 * unit, 8 * unit))


def xl_scores():
    seq, mem, streams, batch, heads, d = 512, 384, 2, 1, 16, 64
    rows, klen, H = streams * seq, mem + seq, heads * d
    bf = torch.bfloat16
    r = lambda *sh: torch.randn(*sh, device="cuda").to(bf)
    q, kv, kr, dvec = r(rows, batch, H), r(klen, batch, 2 * H), r(klen + seq, H), r(rows, batch, H)
    seg_emb = torch.randn(2, H, device="cuda")
    biases = [torch.randn(H, device="cuda") for _ in range(3)]
    masks = (torch.rand(rows, klen, batch, device="cuda") < 0.3).float()
    seg = (torch.rand(seq, klen, batch, device="cuda") < 0.4).to(torch.uint8)
    meta, nseg = ops.xlnet_scores_pack(seq, rows, klen, batch, masks, seg)
    dbd = torch.zeros(batch * heads, rows, klen + seq, dtype=bf, device="cuda")
    for _ in range(5):
        qw, qr, qs, de = ops.xlnet_bias_q(q, biases[0], biases[1], biases[2], seg_emb, heads)
        p = ops.xlnet_scores_fwd(qw, qr, de, kv, kr, seq, heads, 0.125, meta)
        ops.xlnet_scores_bwd(kv, p, dvec, seq, heads, 0.125, meta, nseg, dbd)
    torch.cuda.synchronize()
    n = batch * heads * rows * klen
    print("xl_bias_q_de_kernel: %d bytes per launch (read q, write qw, qr, qs)" % (8 * rows * batch * H))
    print("xl_scores_fwd_kernel: %d bytes per launch (write p; operands %d), %d FLOP (q k^T and the 9/8 window of q kr^T)"
          % (2 * n, 2 * (3 * rows * batch * H + klen * batch * H + (klen + seq) * H), int(2 * 2.125 * n * d)))
    print("xl_scores_bwd_kernel: %d bytes per launch (read p, write ds and the band of dbd), %d FLOP (dvec v^T)" % (6 * n, 2 * n * d))


def elementwise():
    bf = torch.bfloat16
    rows, h, f = 1024, 1024, 4096
    r = torch.randn
    x, dy = r(rows, h, device="cuda").to(bf), r(rows, h, device="cuda").to(bf)
    g, b = torch.ones(h, device="cuda"), torch.zeros(h, device="cuda")
    dg, db, dc = (torch.zeros(h, device="cuda") for _ in range(3))
    big = r(4 * rows, f, device="cuda").to(bf)
    out = torch.zeros(f, device="cuda")
    n_acc = 12596224                     # parameters of one encoder layer
    acc, grad = torch.zeros(n_acc, device="cuda"), torch.ones(n_acc, device="cuda")
    src = r(h * f, device="cuda")
    xf, dyf = x.float(), dy.float()
    for _ in range(5):
        y, st = ops.layernorm_fwd(x, g, b, 1e-12)
        ops.layernorm_bwd(dy, x, g, st, dg, db, dc)
        y16, y32, stf = ops.layernorm_fwd_mixed(xf, g, b, 1e-12)
        ops.layernorm_bwd_mixed(dyf, xf, g, stf, dg, db, dc)
        dx16, dx32, dy16 = ops.layernorm_bwd_mixed(dyf, xf, g, stf, want_dy_bf16=True)
        ops.layernorm_param_grads_mixed(dy16, xf, stf, dg, db, dx16, dc)
        ops.colsum_accum(big, out)
        ops.grad_accumulate(acc, grad)
        ops.cast_to_bf16(src)
    torch.cuda.synchronize()
    e = 2
    print("layernorm_fwd_kernel<bf16>  [%d,%d]: %d bytes per launch (read x, write y)" % (rows, h, 2 * rows * h * e))
    print("layernorm_bwd_kernel<bf16>  [%d,%d]: %d bytes per launch (read dy, x, write dx)" % (rows, h, 3 * rows * h * e))
    print("layernorm_fwd_mixed_kernel  [%d,%d]: %d bytes per launch (read x fp32, write y bf16 + fp32)" % (rows, h, 10 * rows * h))
    print("layernorm_bwd_mixed_kernel  [%d,%d]: %d bytes per launch (read dy, x fp32, write dx bf16 + fp32)" % (rows, h, 14 * rows * h))
    print("layernorm_bwd_mixed_rows_kernel [%d,%d]: %d bytes per launch (as above + the bf16 copy of dy)" % (rows, h, 16 * rows * h))
    print("layernorm_param_grad_mixed_kernel [%d,%d]: %d bytes per launch (read dy bf16, x fp32, dx bf16)" % (rows, h, 8 * rows * h))
    print("colsum_kernel<bf16>         [%d,%d]: %d bytes per launch (read x)" % (4 * rows, f, 4 * rows * f * e))
    print("accumulate_kernel<float>    %d elements: %d bytes per launch (read acc, g, write acc)" % (n_acc, 12 * n_acc))
    print("cast_kernel<bf16,float>     %d elements: %d bytes per launch (read fp32, write bf16)" % (h * f, 6 * h * f))


def timeline(workload):
    import types
    import bench
    from dapple_amd import synthetic
    args = types.SimpleNamespace(wgrad_group=8, bf16_residual_stream=False, pair_passes=False, xlnet_attention="auto")
    c = dict(synthetic.CONFIGS[workload])
    wl = bench.MAKERS[c["kind"]](c, args)
    stage = wl.stage
    if stage.overlap_supported():
        stage.enable_overlap()
    for _ in range(3):
        wl.step()
    torch.cuda.synchronize()
    probe = torch.cuda.Stream()
    plain_backward = stage.backward
    marks = []

    def backward(slot, d_out, d_in=None, ready=False):
        plain_backward(slot, d_out, d_in, ready=ready)
        stage.wait_backward(slot, probe)
        e = torch.cuda.Event(enable_timing=True)
        e.record(probe)
        marks.append(e)
    stage.backward = backward
    plain_forward = stage.forward
    fmarks = []

    def forward(*a, **k):
        r = plain_forward(*a, **k)
        e = torch.cuda.Event(enable_timing=True)
        e.record()     # the forward passes run on the stream the step is queued on
        fmarks.append(e)
        return r
    stage.forward = forward
    for _ in range(3):
        marks.clear()
        fmarks.clear()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e0.record()
        t0 = time.perf_counter()
        wl.step()
        e1 = torch.cuda.Event(enable_timing=True)
        e1.record()
        host = time.perf_counter() - t0
        torch.cuda.synchronize()
        tot = e0.elapsed_time(e1)
        ts = [e0.elapsed_time(e) for e in marks]
        print("%s: step %.2f ms (the host queued it in %.2f ms); backward chains end at %s ms" % (workload, tot, host * 1e3, " ".join("%.2f" % t for t in ts)))
        print("   forward passes end at %s ms" % " ".join("%.2f" % e0.elapsed_time(e) for e in fmarks))
        print("   from one chain's end to the next: %s ms; after the last chain: %.2f ms"
              % (" ".join("%.2f" % (b - a) for a, b in zip([0.0] + ts[:-1], ts)), tot - ts[-1]))


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "timeline":
        timeline(sys.argv[2] if len(sys.argv) > 2 else "bert48_half")
    elif len(sys.argv) > 1 and sys.argv[1] == "gemms":
        gemms()
    elif len(sys.argv) > 1 and sys.argv[1] == "elementwise":
        elementwise()
    elif len(sys.argv) > 1 and sys.argv[1] == "attention":
        attention()
    elif len(sys.argv) > 1 and sys.argv[1] == "xl_scores":
        xl_scores()
    elif len(sys.argv) > 1 and sys.argv[1] == "gemm_table":
        gemm_table()
    elif len(sys.argv) > 1 and sys.argv[1] == "grouped":
        grouped()
    elif len(sys.argv) > 1 and sys.argv[1] == "wgrad_group":
        wgrad_group()
    else:
        accumulate(int(sys.argv[2]) if len(sys.argv) > 2 else 1 << 26)
