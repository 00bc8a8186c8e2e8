"""Benchmark of the pipeline-stage hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload bert48_half] [--no-cpu-baseline]

One step = the whole early-backward (1F1B) pass of one stage over its M micro-batches: refresh
the compute copies of the fp32 master weights, zero the master gradients, then M forwards and M
backwards in schedule order with in-place fp32 gradient accumulation.  Inputs, weights and
upstream gradients are synthetic, seeded and already resident in HBM.  Prints ONE JSON line.

Workloads (BASELINE.json configs): bert48_half (configs[3], the one the metric is quoted on and
the default), bert_large_2l (configs[0]), vgg19_stage0 (configs[1]), gnmt16_encoder (configs[2]),
xlnet36_half (configs[4]).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"bf16": 2.5e15, "fp32": 157.3e12, "hbm": 8.0e12}  # MI355X dense MFMA FLOP/s and HBM B/s


def host_cores():
    cores = os.cpu_count() or 1
    try:
        cores = min(cores, len(os.sched_getaffinity(0)))
    except Exception:
        pass
    return min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))


# ------------------------------------------------------------------------------------------ workloads
class Workload:
    """step(): one stage step on the GPU; cpu_baseline(): (seconds, samples, description) of the fp32
    torch-CPU restatement on a bounded sample of the same workload."""


def make_bert(c, args):
    import torch
    from dapple_amd import runtime, synthetic
    B, S, H, F, N, L, M = c["micro_batch"], c["seq"], c["hidden"], c["ffn"], c["heads"], c["num_layers"], c["num_micro_batches"]
    adt = torch.bfloat16 if c["dtype"] == "bf16" else torch.float32
    K = runtime.stash_depth(0, 2)
    G = max(1, min(args.wgrad_group, M))
    stage = runtime.bert_stage(L, H, N, F, B, S, c["dtype"], stash_slots=K, embeddings=c["embeddings"], wgrad_group=G,
                               residual_fp32=not args.bf16_residual_stream)
    stage.bind(synthetic.bert_weights(synthetic.SEED_WEIGHT + c["index"], L, H, F, embeddings=c["embeddings"]))
    if c["embeddings"] is None:
        xs = [torch.as_tensor(x).cuda().to(adt) for x in synthetic.bert_activation_inputs(synthetic.SEED_INPUT + c["index"], M, B, S, H)]
        dxs = [torch.empty(B * S, H, dtype=adt, device="cuda") for _ in range(M)]
    else:
        xs = [torch.as_tensor(x).cuda() for x in synthetic.bert_id_inputs(synthetic.SEED_INPUT + c["index"], M, B, S, c["embeddings"][0])]
        dxs = None
    dys = [torch.as_tensor(x).cuda().to(adt) for x in synthetic.upstream_grads(synthetic.SEED_GRAD + c["index"], M, (B * S, H))]
    outs = [torch.empty(B * S, H, dtype=adt, device="cuda") for _ in range(M)]
    rt = runtime.StageRuntime(stage, 0, 2, M, pair_passes=args.pair_passes)
    wl = Workload()
    wl.stage = stage
    wl.step = lambda: (stage.refresh_weights(), stage.zero_grads(), rt.step(xs, dys, outs, dxs))
    wl.samples = B * M
    fwd = 2 * S * (4 * H * H + 2 * H * F) + 4 * S * S * H
    wl.flops_per_sample = 3 * fwd * L
    wl.config = {"layers": L, "hidden": H, "heads": N, "ffn": F, "seq": S, "micro_batch": B, "micro_batches": M,
                 "embedding": c["embeddings"] is not None, "schedule": "1F1B stage 0 of 2, stash K=%d" % K,
                 "wgrad_group": G, "residual_stream": "fp32" if (c["dtype"] != "bf16" or not args.bf16_residual_stream) else "bf16",
                 "pair_passes": args.pair_passes}

    def cpu():
        from oracle import bert as ob
        Lt = min(L, 24)
        w = ob.to_torch(synthetic.bert_weights(synthetic.SEED_WEIGHT + c["index"], Lt, H, F, embeddings=c["embeddings"]),
                        torch.float32, requires_grad=True)
        x = xs[0].cpu() if c["embeddings"] is not None else xs[0].cpu().float()
        dy = dys[0].cpu().float()
        ob.stage_vjp(x, w, dy, [0], B, S, N)
        t0 = time.perf_counter()
        ob.stage_vjp(x, w, dy, list(range(Lt)), B, S, N)
        dt = time.perf_counter() - t0
        return dt, B, "1 of %d micro-batches (%d samples) fwd+bwd through all %d layers" % (M, B, Lt)
    wl.cpu = cpu
    return wl


def make_vgg(c, args):
    import torch
    from dapple_amd import runtime, synthetic
    B, M, layers = c["micro_batch"], c["num_micro_batches"], c["layers"]
    Hh, Ww, Cin = c["height"], c["width"], c["in_channels"]
    K = runtime.stash_depth(0, 2, "2S-1")
    stage = runtime.vgg_stage(layers, B, Hh, Ww, Cin, stash_slots=K)
    stage.bind(synthetic.vgg_weights(synthetic.SEED_WEIGHT + c["index"], layers, Cin))
    xs = [torch.as_tensor(x).cuda() for x in synthetic.vgg_inputs(synthetic.SEED_INPUT + c["index"], M, B, Hh, Ww, Cin)]
    dys = [torch.as_tensor(x).cuda() for x in synthetic.upstream_grads(synthetic.SEED_GRAD + c["index"], M, stage.out_shape)]
    outs = [torch.empty(stage.out_shape, device="cuda") for _ in range(M)]
    rt = runtime.StageRuntime(stage, 0, 2, M, variant="2S-1", needs_input_grad=False)
    wl = Workload()
    wl.stage = stage
    wl.step = lambda: (stage.refresh_weights(), stage.zero_grads(), rt.step(xs, dys, outs))
    wl.samples = B * M
    macs, h, w_, cin, first = 0, Hh, Ww, Cin, None
    for _, cout in layers:
        if cout is None:
            h, w_ = h // 2, w_ // 2
        else:
            m = h * w_ * 9 * cin * cout
            first = m if first is None else first
            macs += m
            cin = cout
    wl.flops_per_sample = 2 * (3 * macs - first)       # no input gradient through the first conv
    wl.config = {"convs": sum(1 for _, c_ in layers if c_), "pools": sum(1 for _, c_ in layers if c_ is None),
                 "image": [Hh, Ww, Cin], "micro_batch": B, "micro_batches": M, "schedule": "1F1B (2S-1 variant) stage 0 of 2, stash K=%d" % K}

    def cpu():
        from oracle import vgg as ov
        nb = 4
        w = ov.to_torch(synthetic.vgg_weights(synthetic.SEED_WEIGHT + c["index"], layers, Cin), torch.float32, requires_grad=True)
        x, dy = xs[0][:nb].cpu(), dys[0][:nb].cpu()
        t0 = time.perf_counter()
        ov.stage_vjp(x, w, dy, layers)
        dt = time.perf_counter() - t0
        return dt, nb, "%d of %d images of one micro-batch, fwd+bwd through all %d ops" % (nb, B, len(layers))
    wl.cpu = cpu
    return wl


def make_vgg_last(c, args):
    """The last device of the sliced VGG19 (K = 1): conv tail, classification block, loss, backward down to the boundary."""
    import numpy as np
    import torch
    from dapple_amd import ops, runtime, synthetic
    B, M, layers = c["micro_batch"], c["num_micro_batches"], c["layers"]
    Hh, Ww, Cin, FC, CL = c["height"], c["width"], c["in_channels"], c["fc"], c["classes"]
    stage = runtime.vgg_stage(layers, B, Hh, Ww, Cin, stash_slots=1, need_input_grad=True)
    stage.bind(synthetic.vgg_weights(synthetic.SEED_WEIGHT + c["index"], layers, Cin))
    feat = 1
    for d in stage.out_shape[1:]:
        feat *= d
    hw = {k: torch.as_tensor(v).cuda() for k, v in synthetic.vgg_head_weights(synthetic.SEED_WEIGHT + c["index"] + 1, feat, FC, CL).items()}
    hg = {k: torch.zeros_like(v) for k, v in hw.items()}
    r = np.random.Generator(np.random.PCG64(synthetic.SEED_INPUT + c["index"]))
    xs = [torch.as_tensor(np.abs(r.standard_normal((B, Hh, Ww, Cin))).astype(np.float32)).cuda() for _ in range(M)]
    labels = [torch.as_tensor(r.integers(0, CL, B).astype(np.float32)).cuda() for _ in range(M)]
    y = torch.empty(stage.out_shape, device="cuda")
    dxs = [torch.empty(B, Hh, Ww, Cin, device="cuda") for _ in range(M)]

    def step():
        stage.refresh_weights(); stage.zero_grads()
        for g in hg.values():
            g.zero_()
        for j in range(M):
            stage.forward(0, xs[j], y)
            _, _, dy = ops.vgg_head(y.reshape(B, feat), hw, labels[j], grads=hg, loss_mode="sparse_ce")
            stage.backward(0, dy.reshape(stage.out_shape), dxs[j])
    wl = Workload()
    wl.stage = stage
    wl.step = step
    wl.samples = B * M
    macs, h, w_, cin = 0, Hh, Ww, Cin
    for _, cout in layers:
        if cout is None:
            h, w_ = h // 2, w_ // 2
        else:
            macs += h * w_ * 9 * cin * cout
            cin = cout
    wl.flops_per_sample = 2 * 3 * (macs + feat * FC + FC * FC + FC * CL)
    wl.config = {"convs": sum(1 for _, c_ in layers if c_), "boundary": [Hh, Ww, Cin], "fc": FC, "classes": CL, "micro_batch": B,
                 "micro_batches": M, "loss": "sparse cross entropy",
                 "schedule": "last stage (K=1): forward, classification block + loss, backward per micro-batch"}

    def cpu():
        from oracle import vgg as ov
        nb = 8
        w = ov.to_torch({**synthetic.vgg_weights(synthetic.SEED_WEIGHT + c["index"], layers, Cin),
                         **{k: v.cpu().numpy() for k, v in hw.items()}}, torch.float32, requires_grad=True)
        x = xs[0][:nb].cpu().requires_grad_(True)
        t0 = time.perf_counter()
        loss = ov.head_loss(ov.head_forward(ov.stage_forward(x, w, layers).reshape(nb, -1), w), labels[0][:nb].cpu(), "sparse_ce")
        torch.autograd.grad(loss, [x] + list(w.values()))
        dt = time.perf_counter() - t0
        return dt, nb, "%d of %d images of one micro-batch, conv tail + classification block + loss, fwd+bwd" % (nb, B)
    wl.cpu = cpu
    return wl


def make_gnmt(c, args):
    import torch
    from dapple_amd import runtime, synthetic
    L, U, V, B, T, M = c["num_layers"], c["units"], c["vocab"], c["micro_batch"], c["seq"], c["num_micro_batches"]
    K = runtime.stash_depth(0, 2)
    stage = runtime.gnmt_stage(L, U, V, B, T, stash_slots=K, forget_bias=c["forget_bias"])
    stage.bind(synthetic.gnmt_weights(synthetic.SEED_WEIGHT + c["index"], L, U, V))
    ids = [torch.as_tensor(x).cuda() for x in synthetic.gnmt_id_inputs(synthetic.SEED_INPUT + c["index"], M, B, T, V)]
    dys = [torch.as_tensor(x).cuda() for x in synthetic.upstream_grads(synthetic.SEED_GRAD + c["index"], M, (T, B, U))]
    outs = [torch.empty(T, B, U, device="cuda") for _ in range(M)]
    rt = runtime.StageRuntime(stage, 0, 2, M)
    wl = Workload()
    wl.stage = stage
    wl.step = lambda: (stage.refresh_weights(), stage.zero_grads(), rt.step(ids, dys, outs))
    wl.samples = B * M
    per_token = 2 * 4 * U * (2 * (U + U) + (2 * U + U) + (L - 2) * (U + U))
    wl.flops_per_sample = 3 * per_token * T
    wl.config = {"layers": L, "units": U, "vocab": V, "seq": T, "micro_batch": B, "micro_batches": M,
                 "schedule": "1F1B stage 0 of 2, stash K=%d" % K}

    def cpu():
        from oracle import gnmt as og
        nb = 16
        w = og.to_torch(synthetic.gnmt_weights(synthetic.SEED_WEIGHT + c["index"], L, U, V), torch.float32, requires_grad=True)
        t0 = time.perf_counter()
        og.stage_vjp(ids[0][:nb].cpu(), w, dys[0][:, :nb].cpu().contiguous(), L, c["forget_bias"])
        dt = time.perf_counter() - t0
        return dt, nb, "%d of %d sequences of one micro-batch, fwd+BPTT through all %d layers" % (nb, B, L)
    wl.cpu = cpu
    return wl


def make_gnmt_attention(c, args):
    """Decoder cell 0 under the attention wrapper (device 0, behind the encoder): memory in, cell outputs out."""
    import numpy as np
    import torch
    from dapple_amd import runtime, synthetic
    U, V, B, T, S, M = c["units"], c["vocab"], c["micro_batch"], c["seq"], c["src_seq"], c["num_micro_batches"]
    K = runtime.stash_depth(0, 2)
    stage = runtime.gnmt_attention_stage(U, V, B, T, S, stash_slots=K, forget_bias=c["forget_bias"])
    stage.bind(synthetic.gnmt_attention_weights(synthetic.SEED_WEIGHT + c["index"], U, V))
    r = np.random.Generator(np.random.PCG64(synthetic.SEED_INPUT + c["index"]))
    mems = [torch.as_tensor(r.standard_normal((S, B, U)).astype(np.float32)).cuda() for _ in range(M)]
    ids = [torch.as_tensor(x).cuda() for x in synthetic.gnmt_id_inputs(synthetic.SEED_INPUT + c["index"], M, B, T, V)]
    lens = [torch.as_tensor(r.integers(S // 2, S + 1, B).astype(np.int32)).cuda() for _ in range(M)]
    dys = [torch.as_tensor(x).cuda() for x in synthetic.upstream_grads(synthetic.SEED_GRAD + c["index"], M, (T, B, U))]
    outs = [torch.empty(T, B, U, device="cuda") for _ in range(M)]
    dmems = [torch.empty(S, B, U, device="cuda") for _ in range(M)]
    rt = runtime.StageRuntime(stage, 0, 2, M)
    wl = Workload()
    wl.stage = stage
    wl.step = lambda: (stage.refresh_weights(), stage.zero_grads(),
                       rt.step(mems, dys, outs, dmems, before_forward=lambda slot, j: stage.set_decoder_inputs(slot, ids[j], lens[j])))
    wl.samples = B * M
    # per target step: cell (3U x 4U), query layer (U x U), scores and context over the source (2 S U); once: keys (S U U)
    wl.flops_per_sample = 3 * (T * 2 * (3 * U * 4 * U + U * U + 2 * S * U) + 2 * S * U * U)
    wl.config = {"units": U, "vocab": V, "seq": T, "src_seq": S, "micro_batch": B, "micro_batches": M,
                 "schedule": "1F1B stage 0 of 2, stash K=%d" % K}

    def cpu():
        from oracle import gnmt as og
        nb = 16
        w = {k: torch.tensor(v, dtype=torch.float32) for k, v in synthetic.gnmt_attention_weights(synthetic.SEED_WEIGHT + c["index"], U, V).items()}
        w[og.ATT_G] = w[og.ATT_G].reshape(())
        w = {k: v.requires_grad_(True) for k, v in w.items()}
        mem = mems[0][:, :nb].cpu().contiguous().requires_grad_(True)
        t0 = time.perf_counter()
        out, _ = og.attention_cell_forward(ids[0][:nb].cpu(), mem, lens[0][:nb].cpu(), w, c["forget_bias"])
        torch.autograd.grad(out, [mem] + list(w.values()), grad_outputs=dys[0][:, :nb].cpu().contiguous(), allow_unused=True)
        dt = time.perf_counter() - t0
        return dt, nb, "%d of %d sequences of one micro-batch, fwd+BPTT" % (nb, B)
    wl.cpu = cpu
    return wl


def make_gnmt_decoder(c, args):
    """Decoder cells 1.. + output projection + loss (device 1, the last stage: K = 1, every forward is followed by its loss
    and its backward pass)."""
    import numpy as np
    import torch
    from dapple_amd import ops, runtime, synthetic
    L, F0, U, V, B, T, M = c["num_layers"], c["first_layer"], c["units"], c["vocab"], c["micro_batch"], c["seq"], c["num_micro_batches"]
    stage = runtime.gnmt_decoder_stage(L, U, B, T, stash_slots=1, first_layer=F0, forget_bias=c["forget_bias"])
    stage.bind(synthetic.gnmt_decoder_weights(synthetic.SEED_WEIGHT + c["index"], F0, L, U))
    r = np.random.Generator(np.random.PCG64(synthetic.SEED_INPUT + c["index"]))
    xs = [torch.as_tensor(r.standard_normal((T, B, U)).astype(np.float32)).cuda() for _ in range(M)]
    proj = torch.as_tensor(r.uniform(-0.1, 0.1, (U, V)).astype(np.float32)).cuda()
    dproj = torch.zeros_like(proj)
    tgt = [torch.as_tensor(x).cuda() for x in synthetic.gnmt_id_inputs(synthetic.SEED_GRAD + c["index"], M, B, T, V)]
    lens = [torch.as_tensor(r.integers(T // 2, T + 1, B).astype(np.int32)).cuda() for _ in range(M)]
    y = torch.empty(T, B, U, device="cuda")
    dxs = [torch.empty(T, B, U, device="cuda") for _ in range(M)]

    def step():
        stage.refresh_weights(); stage.zero_grads(); dproj.zero_()
        for j in range(M):
            stage.forward(0, xs[j], y)
            _, dy = ops.nmt_loss_head(y, proj, tgt[j], lens[j], d_proj_kernel=dproj)
            stage.backward(0, dy, dxs[j])
    wl = Workload()
    wl.stage = stage
    wl.step = step
    wl.samples = B * M
    wl.flops_per_sample = 3 * T * (L * 2 * 3 * U * 4 * U + 2 * U * V)
    wl.config = {"layers": L, "first_layer": F0, "units": U, "vocab": V, "seq": T, "micro_batch": B, "micro_batches": M,
                 "schedule": "last stage (K=1): forward, projection + loss, backward per micro-batch"}

    def cpu():
        from oracle import gnmt as og
        nb = 8
        w = og.to_torch(synthetic.gnmt_decoder_weights(synthetic.SEED_WEIGHT + c["index"], F0, L, U), torch.float32, requires_grad=True)
        k = proj.cpu().requires_grad_(True)
        x = xs[0][:, :nb].cpu().contiguous().requires_grad_(True)
        t0 = time.perf_counter()
        loss, _ = og.nmt_loss(og.decoder_part2_forward(x, None, w, F0, L, c["forget_bias"]), k, tgt[0][:nb].cpu(), lens[0][:nb].cpu())
        torch.autograd.grad(loss, [x, k] + list(w.values()))
        dt = time.perf_counter() - t0
        return dt, nb, "%d of %d sequences of one micro-batch, fwd+BPTT through all %d cells, projection and loss" % (nb, B, L)
    wl.cpu = cpu
    return wl


def make_xlnet(c, args):
    import numpy as np
    import torch
    from dapple_amd import runtime, synthetic
    L, H, N, F, B, Q, Mm, S, M = (c["num_layers"], c["hidden"], c["heads"], c["ffn"], c["micro_batch"], c["seq"], c["mem_len"],
                                  c["streams"], c["num_micro_batches"])
    adt = torch.bfloat16 if c["dtype"] == "bf16" else torch.float32
    K = runtime.stash_depth(0, 2)
    G = max(1, min(args.wgrad_group, M)) if c["dtype"] == "bf16" else 1
    stage = runtime.xlnet_stage(L, H, N, F, B, Q, c["dtype"], stash_slots=K, mem_len=Mm, streams=S,
                                attention=args.xlnet_attention, residual_fp32=not args.bf16_residual_stream, wgrad_group=G)
    stage.bind(synthetic.xlnet_weights(synthetic.SEED_WEIGHT + c["index"], L, H, N, F))
    xs = [torch.as_tensor(np.stack(x)).cuda().to(adt) for x in synthetic.xlnet_stream_inputs(synthetic.SEED_INPUT + c["index"], M, Q, B, H, S)]
    dys = [torch.as_tensor(np.stack(x)).cuda().to(adt) for x in synthetic.xlnet_stream_inputs(synthetic.SEED_GRAD + c["index"], M, Q, B, H, S)]
    outs = [torch.empty(S, Q, B, H, dtype=adt, device="cuda") for _ in range(M)]
    dxs = [torch.empty_like(o) for o in outs]
    masks_np = synthetic.xlnet_perm_masks(90 + c["index"], Q, Mm, B)[:S]
    masks = torch.as_tensor(np.stack(masks_np)).cuda()
    mems_np = synthetic.xlnet_mems(50 + c["index"], L, Mm, B, H)
    mems = torch.as_tensor(np.stack(mems_np)).cuda().to(adt)
    rt = runtime.StageRuntime(stage, 0, 2, M)
    hook = lambda slot, j: stage.set_inputs(slot, masks, None, mems)
    wl = Workload()
    wl.stage = stage
    wl.step = lambda: (stage.refresh_weights(), stage.zero_grads(), rt.step(xs, dys, outs, dxs, before_forward=hook))
    wl.samples = B * M
    Kl, R = Mm + Q, Mm + 2 * Q
    # per layer fwd: q (S streams), k|v over klen, k_r over rlen, o (S streams), scores/values and position term per stream, FFN
    fwd = 2 * H * H * (S * Q + 2 * Kl + R + S * Q) + S * (2 * 2 * Q * Kl * H + 2 * Q * R * H) + S * 4 * Q * H * F
    wl.flops_per_sample = 3 * fwd * L
    wl.config = {"layers": L, "hidden": H, "heads": N, "ffn": F, "seq": Q, "mem_len": Mm, "streams": S, "micro_batch": B,
                 "micro_batches": M, "schedule": "1F1B stage 0 of 2, stash K=%d" % K, "flops": "two-stream count", "wgrad_group": G,
                 "residual_stream": "fp32" if (c["dtype"] != "bf16" or not args.bf16_residual_stream) else "bf16",
                 "attention_scores": "one kernel per pass" if args.xlnet_attention == "auto" else "separate launches, fp32 scores"}

    def cpu():
        from oracle import xlnet as ox
        Lt = 4
        w = ox.to_torch(synthetic.xlnet_weights(synthetic.SEED_WEIGHT + c["index"], Lt, H, N, F), torch.float32, requires_grad=True)
        streams = [xs[0][s].cpu().float() for s in range(S)]
        d_outs = [dys[0][s].cpu().float() for s in range(S)]
        mm = [torch.as_tensor(m) for m in mems_np[:Lt]]
        mk = [torch.as_tensor(m) for m in masks_np]
        t0 = time.perf_counter()
        ox.stage_vjp(streams, mm, w, d_outs, list(range(Lt)), N, mk, torch.zeros(Q, B, dtype=torch.int64))
        dt = time.perf_counter() - t0
        return dt * L / Lt, B, "1 of %d micro-batches (%d sample) fwd+bwd through %d of %d layers, scaled to %d" % (M, B, Lt, L, L)
    wl.cpu = cpu
    return wl


# HBM bytes per launch come from rocprofv3 --pmc runs (counters cannot be read from inside this process): the committed
# summary of those runs holds one machine-readable row per GEMM shape of the headline workload's layer.
TRAFFIC_SOURCE = "profiles/gemm_bert48_layer_hbm_traffic.txt"


def traffic_rows(path=None):
    """[(kernel tag, shape name, (m, n, k), bytes read, bytes written, algorithmic bytes)] of the rows 'traffic | ...'."""
    path = path or os.path.join(os.path.dirname(os.path.abspath(__file__)), TRAFFIC_SOURCE)
    rows = []
    if not os.path.exists(path):
        return rows
    with open(path) as f:
        for line in f:
            if line.startswith("traffic |"):
                p = [x.strip() for x in line.split("|")]
                rows.append((p[1], p[2], tuple(int(x) for x in p[3].split("x")), int(p[4]), int(p[5]), int(p[6])))
    return rows


def make_amoeba(c, args):
    import numpy as np
    import torch
    from dapple_amd import amoeba, slices, synthetic
    ops_, idx, used = synthetic.AMOEBA_NORMAL_CELLS[c["cell"]]
    f, cin, B, Hh, Ww, M = c["filters"], c["in_channels"], c["micro_batch"], c["height"], c["width"], c["num_micro_batches"]
    shapes = amoeba.cell_variable_shapes("cell_1", cin, cin, f, ops_, idx, used)
    w_np = synthetic.amoeba_cell_weights(synthetic.SEED_WEIGHT + c["index"], shapes)
    variables = {k: torch.as_tensor(v).cuda() for k, v in w_np.items()}
    grads = {k: torch.zeros_like(v) for k, v in variables.items() if "moving_" not in k}
    cell = slices.BaseCell(f, ops_, used, idx, 1.0, 14, 0).bind(variables, grads)
    rng = np.random.default_rng(synthetic.SEED_INPUT + c["index"])
    nets = [torch.as_tensor(rng.standard_normal((B, Hh, Ww, cin)).astype(np.float32)).cuda() for _ in range(M)]
    prevs = [torch.as_tensor(rng.standard_normal((B, Hh, Ww, cin)).astype(np.float32)).cuda() for _ in range(M)]
    n_out = f * sum(1 for u in used if not u)
    dys = [torch.as_tensor(rng.standard_normal((B, Hh, Ww, n_out)).astype(np.float32)).cuda() for _ in range(M)]

    def step():
        for g in grads.values():
            g.zero_()
        for j in range(M):                      # K = 1: F0 B0 F1 B1 ... (a cell keeps one micro-batch's activations)
            cell(nets[j], scope="cell_1", prev_layer=prevs[j], cell_num=1)
            cell.backward(dys[j])

    class _NoStage:
        def overlap_supported(self):
            return False

        def close(self):
            pass
    wl = Workload()
    wl.stage = _NoStage()
    wl.step = step
    wl.samples = B * M
    rows = Hh * Ww
    flops = 0
    for name, shp in shapes.items():            # every kernel that is a matrix of a GEMM: 2 * rows * cin * cout forward
        if name.endswith("weights") and len(shp) == 2:
            flops += 2 * rows * shp[0] * shp[1]
    wl.flops_per_sample = 3 * flops
    wl.config = {"cell": c["cell"], "filters": f, "in_channels": cin, "map": [Hh, Ww], "micro_batch": B, "micro_batches": M,
                 "schedule": "F0 B0 F1 B1 ... (one micro-batch in flight)", "flops": "the cell's convolutions as GEMMs, x 3 for the backward pass"}

    def cpu():
        from oracle import amoeba as oa
        p = {k: torch.as_tensor(v) for k, v in w_np.items()}
        t0 = time.perf_counter()
        oa.cell_vjp(nets[0].cpu(), prevs[0].cpu(), p, dys[0].cpu(), "cell_1", f, ops_, idx, used)
        return time.perf_counter() - t0, B, "1 of %d micro-batches (%d samples) forward + backward through the cell" % (M, B)
    wl.cpu = cpu
    return wl


def traffic_of(tag, workload, wgrad_group):
    """Mean measured HBM bytes per launch of the kernel `tag` over the shapes it runs per layer of `workload`, or None
    where no counter run covers it (any workload but the headline one; a weight-gradient grouping other than the two
    measured)."""
    if workload != "bert48_half":
        return None
    rows = [r for r in traffic_rows() if r[0] == tag]
    if tag.endswith(",MN,MN>"):   # weight gradients: the row of the grouping in use
        want = {1: "wgrad ffn1 (", 4: "wgrad ffn1 x4 ("}.get(wgrad_group)
        rows = [r for r in rows if want and r[1].startswith(want)]
    if not rows:
        return None
    return sum(r[3] + r[4] for r in rows) / len(rows)


MAKERS = {"amoeba": make_amoeba, "bert": make_bert, "vgg": make_vgg, "vgg_last": make_vgg_last, "gnmt": make_gnmt, "xlnet": make_xlnet, "gnmt_attention": make_gnmt_attention,
          "gnmt_decoder": make_gnmt_decoder}
METRIC = {"bert48_half": "stage samples/sec fwd+bwd+grad-accum, BERT-48 half-stage; MFMA util %"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="bert48_half")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-overlap", action="store_true", help="keep forward and backward passes on one stream")
    ap.add_argument("--bf16-residual-stream", action="store_true",
                    help="BERT / XLNet bf16 workloads: round the residual stream to bf16 too (faster, twice the error at full depth)")
    ap.add_argument("--wgrad-group", type=int, default=8,
                    help="BERT stages: weight gradients of this many backward passes in one GEMM per weight")
    ap.add_argument("--pair-passes", action="store_true",
                    help="BERT stages: issue F(j+1) and B(j) as ONE call that walks both chains level by level, one grouped launch "
                         "per level (ds_stage_forward_backward), instead of two calls on two streams (measured slower: a what-if)")
    ap.add_argument("--xlnet-attention", choices=["auto", "separate"], default="auto",
                    help="XLNet stages: how the attention scores run (ds_xlnet_cfg.fused_attention)")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="default workload only: skip the three-step runs of the other BASELINE configurations that are attached "
                         "to the line as `workloads`")
    ap.add_argument("--micro-batch", type=int, default=None,
                    help="samples per micro-batch instead of the configuration's (a what-if: the headline is the default)")
    ap.add_argument("--micro-batches", type=int, default=None, help="micro-batches per step instead of the configuration's")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs one pipeline stage on ONE GPU; --gpus %d is not supported "
              "(no collectives or sharding are part of it)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from dapple_amd import _lib, synthetic

    c = dict(synthetic.CONFIGS[args.workload])
    reshaped = False
    for key, val in (("micro_batch", args.micro_batch), ("num_micro_batches", args.micro_batches)):
        if val is not None and val != c[key]:
            c[key] = val
            reshaped = True
    dtype = c["dtype"]
    wl = MAKERS[c["kind"]](c, args)
    overlap = not args.no_overlap and wl.stage.overlap_supported()
    if overlap:
        wl.stage.enable_overlap()   # backward passes on a second stream: F(j+K) runs beside B(j+1)

    for _ in range(args.warmup):
        wl.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        wl.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    value = wl.samples / dt

    # per-kernel durations: one more step with HIP events around every launch (same stream)
    _lib.profile(True)
    wl.step()
    torch.cuda.synchronize()
    prof = _lib.profile_dump()
    _lib.profile(False)
    iso = None
    if overlap:
        # the same kernels with the stage back on one stream: durations free of the other streams' traffic
        wl.stage.enable_overlap(False)
        wl.step()
        _lib.profile(True)
        wl.step()
        torch.cuda.synchronize()
        iso = _lib.profile_dump()
        _lib.profile(False)
    total_ms = sum(v[1] for v in prof.values())
    dom = max(prof, key=lambda t: prof[t][1])
    n, ms, work, unit = prof[dom]
    if unit == "FLOP":
        roof = {"bound": "mfma", "achieved": work / (ms * 1e-3) / 1e12, "peak": PEAK[dtype] / 1e12, "unit": "TFLOP/s"}
    else:
        roof = {"bound": "hbm", "achieved": work / (ms * 1e-3) / 1e9, "peak": PEAK["hbm"] / 1e9, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = None if reshaped else traffic_of(dom, args.workload, wl.config.get("wgrad_group", 1))
    if roof["traffic"] is not None:
        roof["traffic_unit"] = "bytes per launch (FETCH_SIZE + WRITE_SIZE, scaled by a known-traffic kernel), see " + TRAFFIC_SOURCE
    roof.update({"kernel": dom, "launches": n, "avg_launch_us": ms * 1e3 / n, "share_of_kernel_time": ms / total_ms})
    if iso is not None and dom in iso:
        n2, ms2, work2, _ = iso[dom]
        rate = work2 / (ms2 * 1e-3) / (1e12 if unit == "FLOP" else 1e9)
        roof["one_stream"] = {"achieved": rate, "frac": rate / roof["peak"], "avg_launch_us": ms2 * 1e3 / n2,
                              "note": "same kernel with forward, backward and weight-gradient work serialised on one stream"}
    stage_flops = wl.flops_per_sample * wl.samples
    roof["stage_achieved_TFLOPs"] = stage_flops / dt / 1e12
    roof["stage_frac_of_mfma_peak"] = stage_flops / dt / PEAK[dtype]
    kernels = {t: {"launches": v[0], "ms": round(v[1], 3),
                   "rate": round(v[2] / (v[1] * 1e-3) / (1e12 if v[3] == "FLOP" else 1e9), 2),
                   "unit": "TFLOP/s" if v[3] == "FLOP" else "GB/s"} for t, v in sorted(prof.items(), key=lambda kv: -kv[1][1])}
    cfg = {"workload": args.workload + (" (micro-batching changed on the command line)" if reshaped else ""), "grad_accum": "fp32 in place", "flops_per_sample": wl.flops_per_sample}
    cfg.update(wl.config)
    cfg["fwd_bwd_overlap"] = overlap
    line = {
        "metric": METRIC.get(args.workload, "stage samples/sec fwd+bwd+grad-accum, %s; MFMA util %%" % args.workload),
        "value": value, "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic", "config": cfg, "roofline": roof, "kernels": kernels,
    }
    cpu = wl.cpu
    wl.stage.close()
    del wl
    torch.cuda.empty_cache()
    if args.workload == "bert48_half" and not reshaped and not args.no_other_workloads:
        # the other BASELINE configurations, a few steps each, in the same process: throughput and whole-stage fraction of
        # the matrix peak of their arithmetic (no CPU legs, no per-kernel timing)
        others = {}
        for name in ("bert_large_2l", "vgg19_stage0", "gnmt16_encoder", "xlnet36_half", "amoeba_net_d_cell"):
            oc = dict(synthetic.CONFIGS[name])
            ow = MAKERS[oc["kind"]](oc, args)
            o_overlap = not args.no_overlap and ow.stage.overlap_supported()
            if o_overlap:
                ow.stage.enable_overlap()
            ow.step()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(3):
                ow.step()
            torch.cuda.synchronize()
            odt = (time.perf_counter() - t1) / 3
            others[name] = {"value": ow.samples / odt, "unit": "samples/s", "ms_per_step": odt * 1e3, "steps": 3, "dtype": oc["dtype"],
                            "stage_frac_of_peak": ow.flops_per_sample * ow.samples / odt / PEAK[oc["dtype"]]}
            ow.stage.close()
            del ow
            torch.cuda.empty_cache()
        line["workloads"] = others
    if not args.no_cpu_baseline:
        cores = host_cores()
        torch.set_num_threads(cores)
        secs, samples, what = 0.0, 0, ""
        while secs < 10.0:          # repeat the bounded sample until it amounts to >= 10 s of CPU work
            t, n_, what = cpu()
            secs += t
            samples += n_
        line["cpu_baseline"] = {"value": samples / secs, "unit": "samples/s", "cores": cores, "kind": "port",
                                "sample": "%s, fp32 torch-CPU restatement, %.1f s" % (what, secs)}
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
