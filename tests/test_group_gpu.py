"""ds_gemm_grouped: several GEMMs in one launch give what ds_gemm gives on each of them."""
import pytest
import torch

from dapple_amd import ops
from dapple_amd._lib import (DS_EPI_ACCUM, DS_EPI_BIAS, DS_EPI_GELU, DS_EPI_GELU_GRAD, DS_EPI_MUL, DS_EPI_OUT_F32, DS_EPI_RESIDUAL,
                             DS_EPI_RESIDUAL_F32, DS_K_MAJOR, DS_MN_MAJOR)

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _problem(gen, m, n, k, am, bm, flags=0):
    dev = "cuda"
    a = (torch.randn((m, k) if am == DS_K_MAJOR else (k, m), generator=gen, device=dev) * 0.5).to(BF)
    b = (torch.randn((n, k) if bm == DS_K_MAJOR else (k, n), generator=gen, device=dev) * 0.5).to(BF)
    p = dict(a=a, b=b, m=m, n=n, k=k, a_major=am, b_major=bm, flags=flags)
    f32_out = bool(flags & (DS_EPI_ACCUM | DS_EPI_OUT_F32))
    p["c"] = (torch.randn(m, n, generator=gen, device=dev) if flags & DS_EPI_ACCUM else torch.zeros(m, n, device=dev)).to(
        torch.float32 if f32_out else BF)
    if flags & DS_EPI_BIAS:
        p["bias"] = torch.randn(n, generator=gen, device=dev)
    if flags & DS_EPI_RESIDUAL:
        r = torch.randn(m, n, generator=gen, device=dev)
        p["residual"] = r if flags & DS_EPI_RESIDUAL_F32 else r.to(BF)
    if flags & DS_EPI_GELU:
        p["c2"] = torch.zeros(m, n, device=dev, dtype=BF)
    if flags & DS_EPI_MUL:
        p["c2"] = torch.randn(m, n, generator=gen, device=dev).to(BF)
    return p


def _clone(p):
    q = dict(p)
    q["c"] = p["c"].clone()
    if p["flags"] & DS_EPI_GELU:
        q["c2"] = p["c2"].clone()
    return q


def _reference(p):
    a = p["a"].double() if p["a_major"] == DS_K_MAJOR else p["a"].double().t()
    b = p["b"].double().t() if p["b_major"] == DS_K_MAJOR else p["b"].double()
    return a @ b


CASES = [
    # the products of one encoder layer of the BERT-48 half-stage at their real shapes, in the pairs a stage holds at once
    [(1024, 4096, 1024, DS_K_MAJOR, DS_MN_MAJOR, DS_EPI_BIAS | DS_EPI_GELU | DS_EPI_GELU_GRAD, 1),
     (1024, 4096, 1024, DS_K_MAJOR, DS_K_MAJOR, DS_EPI_MUL, 2)],
    [(1024, 1024, 4096, DS_K_MAJOR, DS_MN_MAJOR, DS_EPI_BIAS | DS_EPI_RESIDUAL | DS_EPI_RESIDUAL_F32 | DS_EPI_OUT_F32, 3),
     (1024, 1024, 4096, DS_K_MAJOR, DS_K_MAJOR, DS_EPI_RESIDUAL | DS_EPI_RESIDUAL_F32 | DS_EPI_OUT_F32, 2),
     (1024, 4096, 4096, DS_MN_MAJOR, DS_MN_MAJOR, DS_EPI_ACCUM, 0)],
    [(1024, 3072, 1024, DS_K_MAJOR, DS_MN_MAJOR, DS_EPI_BIAS, 2),
     (4096, 1024, 2048, DS_MN_MAJOR, DS_MN_MAJOR, DS_EPI_ACCUM, 1),
     (1024, 1024, 1024, DS_K_MAJOR, DS_K_MAJOR, 0, 3)],
    # ragged edges in every tile shape, one problem alone, the maximum of eight problems
    [(200, 136, 320, DS_K_MAJOR, DS_MN_MAJOR, DS_EPI_BIAS, c) for c in (0, 1, 2, 3)] +
    [(136, 200, 384, DS_K_MAJOR, DS_K_MAJOR, 0, c) for c in (1, 3)] +
    [(328, 72, 576, DS_MN_MAJOR, DS_MN_MAJOR, DS_EPI_ACCUM, c) for c in (0, 2)],
    [(64, 64, 320, DS_K_MAJOR, DS_MN_MAJOR, 0, 3)],
]


@pytest.mark.parametrize("case", range(len(CASES)))
def test_grouped_launch_against_separate_launches(case):
    gen = torch.Generator(device="cuda").manual_seed(100 + case)
    probs = [dict(_problem(gen, m, n, k, am, bm, fl), cfg=cfg) for m, n, k, am, bm, fl, cfg in CASES[case]]
    alone = [_clone(p) for p in probs]
    ops.gemm_grouped(probs)
    for p in alone:
        q = dict(p)
        q.pop("cfg")
        ops.gemm(**q)
    torch.cuda.synchronize()
    for i, (p, q) in enumerate(zip(probs, alone)):
        ref = _reference(p)
        scale = ref.abs().max().item()
        # the same products summed in another tile order: agreement far inside the bf16 bar of 2e-2
        got, want = p["c"].double(), q["c"].double()
        assert (got - want).abs().max().item() <= 1e-2 * scale, "problem %d differs from ds_gemm" % i
        if p["flags"] & DS_EPI_GELU:
            assert (p["c2"].double() - q["c2"].double()).abs().max().item() <= 1e-2 * scale
        if p["flags"] in (0, DS_EPI_OUT_F32):
            assert (got - ref).abs().max().item() <= 8e-3 * scale, "problem %d differs from the float64 product" % i


def test_grouped_launch_rejects_what_it_cannot_run():
    gen = torch.Generator(device="cuda").manual_seed(7)
    ok = dict(_problem(gen, 128, 128, 512, DS_K_MAJOR, DS_MN_MAJOR), cfg=2)
    with pytest.raises(ValueError):
        ops.gemm_grouped([dict(ok, cfg=7)])
    with pytest.raises(ValueError):   # k no longer than the tile ring
        ops.gemm_grouped([dict(_problem(gen, 128, 128, 128, DS_K_MAJOR, DS_MN_MAJOR), cfg=2)])
    with pytest.raises(ValueError):   # fp32 operands
        p = _problem(gen, 128, 128, 512, DS_K_MAJOR, DS_MN_MAJOR)
        p["a"], p["b"], p["c"] = p["a"].float(), p["b"].float(), p["c"].float()
        ops.gemm_grouped([dict(p, cfg=2)])
    with pytest.raises(ValueError):
        ops.gemm_grouped([ok] * 13)           # more tasks than one launch carries
    with pytest.raises(ValueError):   # an operand smaller than its shape says
        ops.gemm_grouped([dict(ok, m=256)])
