"""The score kernels of XLNet's relative attention as operators (ds_xlnet_scores_*), against the formulas of
xlnet/layers/rel_multihead_attn.py:71-115 and the relative shift of xlnet/layers/lambda_funcs.py:85-93 evaluated with torch
in float64 on the same bf16 inputs.  Tolerance: bf16 outputs 1e-2 of the largest reference value (the rounding of the output
itself is 4e-3), fp32 sums 1e-3."""
import numpy as np
import pytest
import torch

from dapple_amd import ops
from util import rel_err

pytestmark = pytest.mark.gpu
D = 64


def make_case(seq, mem, streams, batch, heads, mask_kind, use_seg, seed):
    g = torch.Generator().manual_seed(seed)
    rows, klen, H = streams * seq, mem + seq, heads * D
    r = lambda *s: torch.randn(*s, generator=g)
    t = {"q": r(rows, batch, H), "kv": r(klen, batch, 2 * H), "kr": r(klen + seq, H), "dvec": r(rows, batch, H)}
    t = {k: v.to(torch.bfloat16).cuda() for k, v in t.items()}
    t["seg_emb"] = (0.5 * r(2, H)).cuda()
    biases = [(0.5 * r(H)).cuda() for _ in range(3)]
    t["qw"], t["qr"], t["qs"], t["de"] = ops.xlnet_bias_q(t["q"], biases[0], biases[1], biases[2], t["seg_emb"], heads)
    for name, bias in zip(("qw", "qr", "qs"), biases):      # q + bias, rounded once
        assert torch.equal(t[name], (t["q"].float() + bias).to(torch.bfloat16)), name
    want_de = torch.einsum("ibnd,nd->bni", t["qs"].double().view(rows, batch, heads, D),
                           (t["seg_emb"][1] - t["seg_emb"][0]).double().view(heads, D))
    assert rel_err(t["de"], want_de.cpu())[0] <= 1e-5
    masks = None
    if mask_kind == "random":       # about a third masked, some rows entirely
        masks = (torch.rand(rows, klen, batch, generator=g) < 0.35).float()
        masks[3::7] = 1.0
    elif mask_kind == "causal":
        i = torch.arange(rows).view(rows, 1, 1) % seq
        j = torch.arange(klen).view(1, klen, 1)
        masks = (j > i + mem).float().expand(rows, klen, batch).contiguous()
    seg = (torch.rand(seq, klen, batch, generator=g) < 0.4).to(torch.uint8) if use_seg else None
    t["masks"] = None if masks is None else masks.cuda()
    t["seg"] = None if seg is None else seg.cuda()
    return t, rows, klen


def reference_p(t, seq, heads, scale):
    rows, batch, H = t["qw"].shape
    klen = t["kv"].shape[0]
    f = lambda x: x.double().view(x.shape[0], batch, heads, D)
    k = f(t["kv"][:, :, :H].contiguous())
    ac = torch.einsum("ibnd,jbnd->bnij", f(t["qw"]), k)
    raw = torch.einsum("ibnd,rnd->bnir", f(t["qr"]), t["kr"].double().view(-1, heads, D))          # un-shifted, [b, n, i', r]
    i = torch.arange(rows, device="cuda") % seq
    col = torch.arange(klen, device="cuda").view(1, klen) + seq - i.view(rows, 1)                   # j + seq - i
    bd = torch.gather(raw, 3, col.expand(batch, heads, rows, klen))
    ef = torch.einsum("ibnd,snd->bnis", f(t["qs"]), t["seg_emb"].double().view(2, heads, D))       # [b, n, i', 2]
    score = ac + bd
    if t["seg"] is not None:
        sel = t["seg"][i].permute(2, 0, 1).long()                                                   # [b, i', j]
        score = score + torch.gather(ef, 3, sel.view(batch, 1, rows, klen).expand(batch, heads, rows, klen))
    else:
        score = score + ef[..., :1]
    score = score * scale
    if t["masks"] is not None:
        score = score - 1e30 * t["masks"].double().permute(2, 0, 1).view(batch, 1, rows, klen)
    return torch.softmax(score, -1).view(batch * heads, rows, klen)


CASES = [(32, 16, 2, 2, 2, "random", True), (48, 160, 1, 2, 2, "causal", True), (64, 64, 2, 1, 8, None, False),
         (16, 0, 1, 3, 2, "random", False), (128, 896, 1, 1, 8, "random", True), (512, 384, 2, 1, 16, "random", True)]


@pytest.mark.parametrize("seq,mem,streams,batch,heads,mask_kind,use_seg", CASES)
def test_scores_forward_and_backward(seq, mem, streams, batch, heads, mask_kind, use_seg):
    t, rows, klen = make_case(seq, mem, streams, batch, heads, mask_kind, use_seg, seed=seq + mem)
    scale = 1.0 / np.sqrt(D)
    meta, nseg = ops.xlnet_scores_pack(seq, rows, klen, batch, t["masks"], t["seg"])
    p = ops.xlnet_scores_fwd(t["qw"], t["qr"], t["de"], t["kv"], t["kr"], seq, heads, scale, meta)
    want = reference_p(t, seq, heads, scale)
    mx, l2 = rel_err(p, want.cpu())
    assert mx <= 1e-2 and l2 <= 1e-2, "probabilities: rel max %.3e, l2 %.3e" % (mx, l2)
    assert torch.allclose(p.double().sum(-1), torch.ones_like(want[..., 0]), atol=2e-2)

    # backward from the kernel's own (rounded) probabilities
    ds, dbd, defs = ops.xlnet_scores_bwd(t["kv"], p, t["dvec"], seq, heads, scale, meta, nseg)
    H = heads * D
    v = t["kv"][:, :, H:].double().reshape(klen, batch, heads, D)
    dp = torch.einsum("ibnd,jbnd->bnij", t["dvec"].double().view(rows, batch, heads, D), v).reshape(batch * heads, rows, klen)
    pd = p.double()
    ds_want = scale * pd * (dp - (pd * dp).sum(-1, keepdim=True))
    mx, l2 = rel_err(ds, ds_want.cpu())
    assert mx <= 1e-2 and l2 <= 1e-2, "score gradients: rel max %.3e, l2 %.3e" % (mx, l2)
    # the un-shifted copy: exactly ds inside the band, untouched (zero) outside
    i = torch.arange(rows, device="cuda") % seq
    col = (torch.arange(klen, device="cuda").view(1, klen) + seq - i.view(rows, 1)).expand(batch * heads, rows, klen)
    assert torch.equal(torch.gather(dbd, 2, col), ds)
    outside = torch.ones_like(dbd, dtype=torch.bool).scatter_(2, col, False)
    assert not dbd[outside].any()
    # segment sums of the rounded gradients, with what is left of the row sum spread in proportion to the key counts
    dsd = ds.double()
    if t["seg"] is not None:
        sel = t["seg"][i].permute(2, 0, 1).double().view(batch, 1, rows, klen).expand(batch, heads, rows, klen).reshape(batch * heads, rows, klen)
    else:
        sel = torch.zeros_like(dsd)
    s1, tot, n1 = (dsd * sel).sum(-1), dsd.sum(-1), sel.sum(-1)
    excess = tot / klen
    want_defs = torch.stack([(tot - s1) - excess * (klen - n1), s1 - excess * n1], -1)
    mx, _ = rel_err(defs, want_defs.cpu())
    assert mx <= 1e-3, "segment sums: rel max %.3e" % mx


def test_scores_reject_shapes_outside_the_kernels():
    t, rows, klen = make_case(16, 8, 1, 1, 2, None, False, seed=1)       # klen 24: not a multiple of 16
    with pytest.raises(Exception, match="outside the kernel"):
        ops.xlnet_scores_fwd(t["qw"], t["qr"], t["de"], t["kv"], t["kr"], 16, 2, 0.125)
