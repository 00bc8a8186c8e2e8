"""Benchmark of the pipeline-stage hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload bert48_half] [--no-cpu-baseline]

One step = the whole 1F1B pass of the stage over its M micro-batches: refresh the bf16
compute copies of the fp32 master weights, zero the master gradients, then M forwards
and M backwards in the early-backward order with in-place fp32 gradient accumulation.
Inputs, weights and upstream gradients are synthetic, seeded and already resident in HBM.
Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"bf16": 2.5e15, "fp32": 157.3e12, "hbm": 8.0e12}  # MI355X dense MFMA FLOP/s and HBM B/s


def stage_flops_per_sample(c):
    """fwd+bwd algorithmic FLOPs of one sample: 3 x 2 x MACs of every contraction in the layers."""
    S, H, F = c["seq"], c["hidden"], c["ffn"]
    fwd = 2 * S * (4 * H * H + 2 * H * F) + 4 * S * S * H
    return 3 * fwd * c["num_layers"]


def cpu_baseline(c, layers_timed=None):
    """Times the fp32 torch-CPU restatement of the same stage on the host cores (a baseline only)."""
    import torch
    from dapple_amd import synthetic
    from oracle import bert as ob
    B, S, H, F, N = c["micro_batch"], c["seq"], c["hidden"], c["ffn"], c["heads"]
    L = c["num_layers"] if layers_timed is None else layers_timed
    cores = os.cpu_count() or 1
    try:
        cores = min(cores, len(os.sched_getaffinity(0)))
    except Exception:
        pass
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    w = ob.to_torch(synthetic.bert_weights(synthetic.SEED_WEIGHT + c["index"], L, H, F), torch.float32, requires_grad=True)
    x = torch.as_tensor(synthetic.bert_activation_inputs(synthetic.SEED_INPUT + c["index"], 1, B, S, H)[0])
    dy = torch.as_tensor(synthetic.upstream_grads(synthetic.SEED_GRAD + c["index"], 1, (B * S, H))[0])
    layers = list(range(L))
    ob.stage_vjp(x, w, dy, layers[:1], B, S, N)          # warm-up: one layer
    t0 = time.perf_counter()
    ob.stage_vjp(x, w, dy, layers, B, S, N)
    dt = time.perf_counter() - t0
    dt_full = dt * c["num_layers"] / L
    return {"value": B / dt_full, "unit": "samples/s", "cores": cores, "kind": "port",
            "sample": "1 of %d micro-batches (%d samples) fwd+bwd through %d of %d layers, fp32 torch-CPU restatement, "
                      "%.1f s, scaled to the full stage" % (c["num_micro_batches"], B, L, c["num_layers"], dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="bert48_half")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--layers", type=int, default=None, help="override the layer count (debugging only; marks the line invalid)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs one pipeline stage on ONE GPU; --gpus %d is not supported "
              "(no collectives or sharding are part of it)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from dapple_amd import _lib, runtime, synthetic

    c = dict(synthetic.CONFIGS[args.workload])
    if args.layers is not None:
        c["num_layers"] = args.layers
    dtype = c["dtype"]
    adt = torch.bfloat16 if dtype == "bf16" else torch.float32
    B, S, H, F, N, L, M = c["micro_batch"], c["seq"], c["hidden"], c["ffn"], c["heads"], c["num_layers"], c["num_micro_batches"]
    num_stages, stage_index = 2, 0
    K = runtime.stash_depth(stage_index, num_stages)

    stage = runtime.bert_stage(L, H, N, F, B, S, dtype, stash_slots=K, embeddings=c["embeddings"])
    stage.bind(synthetic.bert_weights(synthetic.SEED_WEIGHT + c["index"], L, H, F, embeddings=c["embeddings"]))
    if c["embeddings"] is None:
        xs = [torch.as_tensor(x).cuda().to(adt) for x in synthetic.bert_activation_inputs(synthetic.SEED_INPUT + c["index"], M, B, S, H)]
        dxs = [torch.empty(B * S, H, dtype=adt, device="cuda") for _ in range(M)]
    else:
        xs = [torch.as_tensor(x).cuda() for x in synthetic.bert_id_inputs(synthetic.SEED_INPUT + c["index"], M, B, S, c["embeddings"][0])]
        dxs = None
    dys = [torch.as_tensor(x).cuda().to(adt) for x in synthetic.upstream_grads(synthetic.SEED_GRAD + c["index"], M, (B * S, H))]
    outs = [torch.empty(B * S, H, dtype=adt, device="cuda") for _ in range(M)]
    rt = runtime.StageRuntime(stage, stage_index, num_stages, M)

    def step():
        stage.refresh_weights()
        stage.zero_grads()
        rt.step(xs, dys, outs, dxs)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    samples = B * M
    value = samples / dt

    # per-kernel durations: one more step with HIP events around every launch (same stream)
    _lib.profile(True)
    step()
    torch.cuda.synchronize()
    prof = _lib.profile_dump()
    _lib.profile(False)
    total_ms = sum(v[1] for v in prof.values())
    dom = max(prof, key=lambda t: prof[t][1])
    n, ms, work, unit = prof[dom]
    if unit == "FLOP":
        peak = PEAK[dtype]
        roof = {"bound": "mfma", "achieved": work / (ms * 1e-3) / 1e12, "peak": peak / 1e12, "unit": "TFLOP/s"}
    else:
        peak = PEAK["hbm"]
        roof = {"bound": "hbm", "achieved": work / (ms * 1e-3) / 1e9, "peak": peak / 1e9, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = None
    roof["kernel"] = dom
    roof["launches"] = n
    roof["avg_launch_us"] = ms * 1e3 / n
    roof["share_of_kernel_time"] = ms / total_ms
    stage_flops = stage_flops_per_sample(c) * samples
    roof["stage_achieved_TFLOPs"] = stage_flops / dt / 1e12
    roof["stage_frac_of_mfma_peak"] = stage_flops / dt / PEAK[dtype]
    kernels = {t: {"launches": v[0], "ms": round(v[1], 3),
                   "rate": round(v[2] / (v[1] * 1e-3) / (1e12 if v[3] == "FLOP" else 1e9), 2),
                   "unit": "TFLOP/s" if v[3] == "FLOP" else "GB/s"} for t, v in sorted(prof.items(), key=lambda kv: -kv[1][1])}

    line = {
        "metric": "stage samples/sec fwd+bwd+grad-accum, BERT-48 half-stage; MFMA util %",
        "value": value, "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": args.workload + ("" if args.layers is None else "[layers=%d: NOT the baseline config]" % args.layers),
                   "layers": L, "hidden": H, "heads": N, "ffn": F, "seq": S, "micro_batch": B, "micro_batches": M,
                   "schedule": "1F1B stage %d of %d, stash K=%d" % (stage_index, num_stages, K),
                   "grad_accum": "fp32 in place"},
        "roofline": roof,
        "kernels": kernels,
    }
    stage.close()
    del stage
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(c, layers_timed=min(L, 4))
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
