"""Writes the golden fixtures of tests/golden/*.npz from the CPU oracle (fp64).

    python tests/golden/make_fixtures.py

Each file holds, for one reduced-shape case of a BASELINE config: the inputs, the fp32 weights, the
upstream gradients, and the oracle's outputs / input gradients / accumulated weight gradients over all
micro-batches.  Nothing here imports the reference: its own tests hold no numeric vector for this path,
so the fixtures pin the oracle (and through it the HIP stages) against silent drift, not against TF.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from dapple_amd import synthetic  # noqa: E402
from oracle import bert as ob, gnmt as og, vgg as ov, xlnet as ox  # noqa: E402

D = torch.float64


def _acc(acc, dw):
    for k, g in dw.items():
        acc[k] = g.clone() if k not in acc else acc[k] + g


def bert_case():
    L, H, N, F, B, S, M, emb = 2, 32, 4, 64, 2, 8, 3, (50, 2, 16)
    w = synthetic.bert_weights(11, L, H, F, embeddings=emb, stddev=0.1, perturb=True)
    ids = synthetic.bert_id_inputs(12, M, B, S, emb[0])
    dys = synthetic.upstream_grads(13, M, (B * S, H))
    wt = ob.to_torch(w, D, requires_grad=True)
    out, acc = {}, {}
    for m in range(M):
        o, _, dw = ob.stage_vjp(torch.as_tensor(ids[m]), wt, torch.as_tensor(dys[m]).double(), list(range(L)), B, S, N)
        out["out_%d" % m] = o.numpy()
        _acc(acc, dw)
    meta = dict(L=L, H=H, N=N, F=F, B=B, S=S, M=M, vocab=emb[0], type_vocab=emb[1], max_pos=emb[2])
    return meta, w, {"in_%d" % m: ids[m] for m in range(M)}, {"dy_%d" % m: dys[m] for m in range(M)}, out, acc


def vgg_case():
    chans, n, h, w_, cin, M = [32, 32, None, 64], 2, 8, 8, 3, 2
    layers = synthetic.vgg_layers(chans)
    w = synthetic.vgg_weights(21, layers, cin, perturb=True)
    xs = synthetic.vgg_inputs(22, M, n, h, w_, cin)
    dys = synthetic.upstream_grads(23, M, (n, h // 2, w_ // 2, 64))
    wt = ov.to_torch(w, D, requires_grad=True)
    out, acc = {}, {}
    for m in range(M):
        o, _, dw = ov.stage_vjp(torch.as_tensor(xs[m]).double(), wt, torch.as_tensor(dys[m]).double(), layers)
        out["out_%d" % m] = o.numpy()
        _acc(acc, dw)
    meta = dict(n=n, h=h, w=w_, cin=cin, M=M, c0=32, c1=32, c2=64)
    return meta, w, {"in_%d" % m: xs[m] for m in range(M)}, {"dy_%d" % m: dys[m] for m in range(M)}, out, acc


def gnmt_case():
    L, U, V, B, T, M = 3, 16, 20, 4, 5, 2
    w = synthetic.gnmt_weights(31, L, U, V, init_weight=0.4, perturb=True)
    ids = synthetic.gnmt_id_inputs(32, M, B, T, V)
    dys = synthetic.upstream_grads(33, M, (T, B, U))
    wt = og.to_torch(w, D, requires_grad=True)
    out, acc = {}, {}
    for m in range(M):
        o, _, dw = og.stage_vjp(torch.as_tensor(ids[m]), wt, torch.as_tensor(dys[m]).double(), L)
        out["out_%d" % m] = o.numpy()
        _acc(acc, dw)
    return dict(L=L, U=U, V=V, B=B, T=T, M=M), w, {"in_%d" % m: ids[m] for m in range(M)}, \
        {"dy_%d" % m: dys[m] for m in range(M)}, out, acc


def xlnet_case():
    L, H, N, F, B, Q, Mm, S, M = 1, 32, 2, 64, 2, 8, 8, 2, 2
    w = synthetic.xlnet_weights(41, L, H, N, F, stddev=0.2, perturb=True)
    xs = synthetic.xlnet_stream_inputs(42, M, Q, B, H, S)
    dys = synthetic.xlnet_stream_inputs(43, M, Q, B, H, S)
    mems = synthetic.xlnet_mems(44, L, Mm, B, H)
    mh, mg = synthetic.xlnet_perm_masks(45, Q, Mm, B)
    seg = (np.random.Generator(np.random.PCG64(46)).random((Q, B)) > 0.5).astype(np.int64)
    wt = ox.to_torch(w, D, requires_grad=True)
    out, acc = {}, {}
    ins = {"masks": np.stack([mh, mg]), "seg_ids": seg, "mems": np.stack(mems)}
    for m in range(M):
        o, dx, dw = ox.stage_vjp([torch.as_tensor(x).double() for x in xs[m]], [torch.as_tensor(t).double() for t in mems], wt,
                                 [torch.as_tensor(d).double() for d in dys[m]], list(range(L)), N,
                                 [torch.as_tensor(mh).double(), torch.as_tensor(mg).double()], torch.as_tensor(seg))
        out["out_%d" % m] = torch.stack(o).numpy()
        out["dx_%d" % m] = torch.stack(dx).numpy()
        ins["in_%d" % m] = np.stack(xs[m])
        _acc(acc, dw)
    return dict(L=L, H=H, N=N, F=F, B=B, Q=Q, Mm=Mm, S=S, M=M), w, ins, {"dy_%d" % m: np.stack(dys[m]) for m in range(M)}, out, acc


def main():
    for name, fn in (("bert", bert_case), ("vgg", vgg_case), ("gnmt", gnmt_case), ("xlnet", xlnet_case)):
        meta, w, ins, dys, out, acc = fn()
        arrays = {"meta_" + k: np.asarray(v) for k, v in meta.items()}
        arrays.update({"w/" + k: v for k, v in w.items()})
        arrays.update(ins)
        arrays.update(dys)
        arrays.update({k: v.astype(np.float32) for k, v in out.items()})
        arrays.update({"g/" + k: v.numpy().astype(np.float32) for k, v in acc.items()})
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **arrays)
        print(path, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main()
