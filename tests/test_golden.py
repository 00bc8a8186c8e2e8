"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py): the oracle must keep
reproducing them on the CPU, and the HIP stages must match them on the GPU (fp32, 1e-4 relative)."""
import os

import numpy as np
import pytest
import torch

from dapple_amd import synthetic
from oracle import bert as ob, gnmt as og, vgg as ov, xlnet as ox
from util import assert_close

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
D = torch.float64


def load(name):
    z = np.load(os.path.join(GOLD, name + ".npz"))           # allow_pickle stays False
    meta = {k[5:]: int(z[k]) for k in z.files if k.startswith("meta_")}
    w = {k[2:]: z[k] for k in z.files if k.startswith("w/")}
    g = {k[2:]: z[k] for k in z.files if k.startswith("g/")}
    return z, meta, w, g


def _floors(g):
    """Gradients that are zero in exact arithmetic (softmax is invariant to the key bias; one-segment
    XLNet inputs never touch the segment terms) hold only rounding noise: compare them on the scale of
    their non-degenerate sibling."""
    fl = {}
    for k in g:
        if k.endswith("/key/bias"):
            fl[k] = float(np.abs(g[k.replace("/key/", "/query/")]).max())
        if k.endswith("/bias_segment") or k.endswith("/seg_emb"):
            fl[k] = float(np.abs(g[k.rsplit("/", 1)[0] + "/bias_context"]).max())
    return fl


def _check(acc, g, outs, z, tol):
    for m, o in enumerate(outs):
        assert_close(o, z["out_%d" % m], tol, "output mb%d" % m)
    assert set(acc) == set(g)
    fl = _floors(g)
    for k in g:
        assert_close(acc[k].reshape(g[k].shape), g[k], tol, "grad " + k, floor=fl.get(k))


def _sum(acc, dw):
    for k, v in dw.items():
        acc[k] = v.clone() if k not in acc else acc[k] + v


def test_oracle_reproduces_bert_fixture():
    z, c, w, g = load("bert")
    wt = ob.to_torch(w, D, requires_grad=True)
    acc, outs = {}, []
    for m in range(c["M"]):
        o, _, dw = ob.stage_vjp(torch.as_tensor(z["in_%d" % m]), wt, torch.as_tensor(z["dy_%d" % m]).double(),
                                list(range(c["L"])), c["B"], c["S"], c["N"])
        outs.append(o)
        _sum(acc, dw)
    _check(acc, g, outs, z, 1e-6)


def test_oracle_reproduces_vgg_gnmt_xlnet_fixtures():
    z, c, w, g = load("vgg")
    layers = synthetic.vgg_layers([c["c0"], c["c1"], None, c["c2"]])
    wt = ov.to_torch(w, D, requires_grad=True)
    acc, outs = {}, []
    for m in range(c["M"]):
        o, _, dw = ov.stage_vjp(torch.as_tensor(z["in_%d" % m]).double(), wt, torch.as_tensor(z["dy_%d" % m]).double(), layers)
        outs.append(o)
        _sum(acc, dw)
    _check(acc, g, outs, z, 1e-6)

    z, c, w, g = load("gnmt")
    wt = og.to_torch(w, D, requires_grad=True)
    acc, outs = {}, []
    for m in range(c["M"]):
        o, _, dw = og.stage_vjp(torch.as_tensor(z["in_%d" % m]), wt, torch.as_tensor(z["dy_%d" % m]).double(), c["L"])
        outs.append(o)
        _sum(acc, dw)
    _check(acc, g, outs, z, 1e-6)

    z, c, w, g = load("xlnet")
    wt = ox.to_torch(w, D, requires_grad=True)
    masks = [torch.as_tensor(z["masks"][s]).double() for s in range(c["S"])]
    mems = [torch.as_tensor(t).double() for t in z["mems"]]
    acc, outs = {}, []
    for m in range(c["M"]):
        o, dx, dw = ox.stage_vjp([torch.as_tensor(x).double() for x in z["in_%d" % m]], mems, wt,
                                 [torch.as_tensor(d).double() for d in z["dy_%d" % m]], list(range(c["L"])), c["N"], masks,
                                 torch.as_tensor(z["seg_ids"]))
        outs.append(torch.stack(o))
        assert_close(torch.stack(dx), z["dx_%d" % m], 1e-6, "dx")
        _sum(acc, dw)
    _check(acc, g, outs, z, 1e-6)


# ------------------------------------------------------------------------------------------------ GPU
@pytest.mark.gpu
def test_hip_stages_match_the_fixtures():
    from dapple_amd import runtime
    from util import dev
    tol = 1e-4
    # BERT
    z, c, w, g = load("bert")
    M = c["M"]
    st = runtime.bert_stage(c["L"], c["H"], c["N"], c["F"], c["B"], c["S"], "fp32", 2, embeddings=(c["vocab"], c["type_vocab"], c["max_pos"]))
    st.bind(w)
    xs = [dev(z["in_%d" % m]) for m in range(M)]
    dys = [dev(z["dy_%d" % m]) for m in range(M)]
    outs = [torch.empty(c["B"] * c["S"], c["H"], device="cuda") for _ in range(M)]
    runtime.StageRuntime(st, 0, 2, M).step(xs, dys, outs)
    st.sync()
    floor = {k: float(np.abs(g[k.replace("/key/", "/query/")]).max()) for k in g if k.endswith("/key/bias")}
    for m in range(M):
        assert_close(outs[m], z["out_%d" % m], tol, "bert out")
    for k in g:
        assert_close(st.grads[k], g[k], tol, "bert grad " + k, floor=floor.get(k))
    st.close()
    # VGG
    z, c, w, g = load("vgg")
    M = c["M"]
    layers = synthetic.vgg_layers([c["c0"], c["c1"], None, c["c2"]])
    st = runtime.vgg_stage(layers, c["n"], c["h"], c["w"], c["cin"], 3)
    st.bind(w)
    xs = [dev(z["in_%d" % m]) for m in range(M)]
    dys = [dev(z["dy_%d" % m]) for m in range(M)]
    outs = [torch.empty(st.out_shape, device="cuda") for _ in range(M)]
    runtime.StageRuntime(st, 0, 2, M, variant="2S-1", needs_input_grad=False).step(xs, dys, outs)
    st.sync()
    for m in range(M):
        assert_close(outs[m], z["out_%d" % m], tol, "vgg out")
    for k in g:
        assert_close(st.grads[k], g[k], tol, "vgg grad " + k)
    st.close()
    # GNMT
    z, c, w, g = load("gnmt")
    M = c["M"]
    st = runtime.gnmt_stage(c["L"], c["U"], c["V"], c["B"], c["T"], 2)
    st.bind(w)
    xs = [dev(z["in_%d" % m]) for m in range(M)]
    dys = [dev(z["dy_%d" % m]) for m in range(M)]
    outs = [torch.empty(st.out_shape, device="cuda") for _ in range(M)]
    runtime.StageRuntime(st, 0, 2, M).step(xs, dys, outs)
    st.sync()
    for m in range(M):
        assert_close(outs[m], z["out_%d" % m], tol, "gnmt out")
    for k in g:
        assert_close(st.grads[k], g[k], tol, "gnmt grad " + k)
    st.close()
    # XLNet
    z, c, w, g = load("xlnet")
    M = c["M"]
    st = runtime.xlnet_stage(c["L"], c["H"], c["N"], c["F"], c["B"], c["Q"], "fp32", 2, mem_len=c["Mm"], streams=c["S"])
    st.bind(w)
    xs = [dev(z["in_%d" % m]) for m in range(M)]
    dys = [dev(z["dy_%d" % m]) for m in range(M)]
    outs = [torch.empty(st.out_shape, device="cuda") for _ in range(M)]
    dxs = [torch.empty_like(o) for o in outs]
    masks, mems = dev(z["masks"]), dev(z["mems"])
    seg = torch.as_tensor(z["seg_ids"])
    seg_mat = dev(ox.seg_mat_from_ids(seg, c["Mm"]).numpy().astype(np.uint8))
    runtime.StageRuntime(st, 0, 2, M).step(xs, dys, outs, dxs, before_forward=lambda slot, j: st.set_inputs(slot, masks, seg_mat, mems))
    st.sync()
    for m in range(M):
        assert_close(outs[m], z["out_%d" % m], tol, "xlnet out")
        assert_close(dxs[m], z["dx_%d" % m], tol, "xlnet dx")
    for k in g:
        assert_close(st.grads[k], g[k].reshape(st.grads[k].shape), tol, "xlnet grad " + k)
    st.close()
