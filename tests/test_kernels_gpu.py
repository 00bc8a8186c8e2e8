"""Per-kernel parity through the C ABI against fp64 host arithmetic.

Tolerances: fp32 kernels 1e-4 relative (1e-5 where only summation order differs);
bf16 kernels 2e-2 relative to the fp32/fp64 result on the same bf16-rounded inputs.
"""
import math

import numpy as np
import pytest
import torch

from dapple_amd import ops
from dapple_amd._lib import (DS_EPI_ACCUM, DS_EPI_BIAS, DS_EPI_DGELU, DS_EPI_GELU, DS_EPI_OUT_F32, DS_EPI_RELU, DS_EPI_RESIDUAL_F32,
                             DS_EPI_RESIDUAL, DS_K_MAJOR, DS_MN_MAJOR)
from oracle import bert as ob
from util import assert_close, dev, rel_err

pytestmark = pytest.mark.gpu
DT = {"fp32": torch.float32, "bf16": torch.bfloat16}
TOL = {"fp32": 1e-5, "bf16": 1e-2}


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


@pytest.mark.parametrize("n", [0, 1, 5, 1024, 4099, 12596224])
@pytest.mark.parametrize("gdt", ["fp32", "bf16"])
def test_grad_accumulate_bit_exact(n, gdt):
    r = rng(n + 1)
    acc = r.standard_normal(n).astype(np.float32)
    gs = [r.standard_normal(n).astype(np.float32) for _ in range(3)]
    a = dev(acc)
    want = torch.from_numpy(acc.copy())
    for g in gs:
        gd = dev(g, DT[gdt])
        ops.grad_accumulate(a, gd)
        want += gd.cpu().to(torch.float32)          # exact: fp32 add of the same operands, same order
    assert torch.equal(a.cpu(), want)


def test_grad_accumulate_rejects_bad_arguments():
    a = torch.zeros(8, device="cuda")
    with pytest.raises(ValueError):
        ops.grad_accumulate(a, torch.zeros(9, device="cuda"))
    with pytest.raises(ValueError):
        ops.grad_accumulate(a[1:], torch.zeros(7, device="cuda"))       # not 16-byte aligned


def test_cast_round_trip():
    x = dev(rng(3).standard_normal(100003).astype(np.float32))
    b = ops.cast_to_bf16(x)
    assert torch.equal(b.cpu(), x.cpu().to(torch.bfloat16))
    assert torch.equal(ops.cast_to_f32(b).cpu(), b.cpu().to(torch.float32))


SHAPES = [(128, 128, 64), (256, 384, 128), (1024, 1024, 1024), (72, 40, 24), (8, 8, 8), (200, 136, 72), (64, 3072, 256)]


@pytest.mark.parametrize("dt", ["fp32", "bf16"])
@pytest.mark.parametrize("am,bm", [(0, 0), (0, 1), (1, 1), (1, 0)])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_gemm_layouts(dt, am, bm, m, n, k):
    r = rng(m * 7 + n * 3 + k + am * 2 + bm)
    A = r.standard_normal((m, k)).astype(np.float32)
    B = r.standard_normal((n, k)).astype(np.float32)
    a = dev(A if am == DS_K_MAJOR else A.T, DT[dt])
    b = dev(B if bm == DS_K_MAJOR else B.T, DT[dt])
    c = torch.full((m, n), float("nan"), dtype=DT[dt], device="cuda")
    ops.gemm(a, b, c, m, n, k, am, bm)
    Ar = (a if am == DS_K_MAJOR else a.T).cpu().double()
    Br = (b if bm == DS_K_MAJOR else b.T).cpu().double()
    assert_close(c, Ar @ Br.T, TOL[dt], "gemm")


# Shapes that the dispatcher sends to the 512-thread kernels: 128x128 blocks (>= 192 tiles), 256x128 (>= 200), 256x256
# (>= 200), each with ragged edges and the shortest reduction a block shape accepts.
BIG_SHAPES = [(1024, 3072, 1024), (1016, 3064, 320), (3584, 2048, 256), (3576, 1800, 256), (4096, 4096, 512),
              (3992, 4088, 192)]


@pytest.mark.parametrize("am,bm", [(0, 0), (0, 1), (1, 1), (1, 0)])
@pytest.mark.parametrize("m,n,k", BIG_SHAPES)
def test_gemm_wide_blocks(am, bm, m, n, k):
    r = rng(m + n * 5 + k * 11 + am * 2 + bm)
    A = (r.standard_normal((m, k)) * 0.5).astype(np.float32)
    B = (r.standard_normal((n, k)) * 0.5).astype(np.float32)
    a = dev(A if am == DS_K_MAJOR else A.T, torch.bfloat16)
    b = dev(B if bm == DS_K_MAJOR else B.T, torch.bfloat16)
    bias = dev(r.standard_normal(n), torch.float32)
    res = dev(r.standard_normal((m, n)), torch.bfloat16)
    c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    ops.gemm(a, b, c, m, n, k, am, bm, flags=DS_EPI_BIAS | DS_EPI_RESIDUAL, bias=bias, residual=res, alpha=0.25)
    Ar = (a if am == DS_K_MAJOR else a.T).float()
    Br = (b if bm == DS_K_MAJOR else b.T).float()
    ref = (0.25 * (Ar @ Br.T) + bias + res.float()).cpu().double()   # fp32 on the device: the fp64 host product takes minutes
    assert_close(c, ref, TOL["bf16"], "gemm, wide blocks")
    acc0 = dev(r.standard_normal((m, n)), torch.float32)
    acc = acc0.clone()
    ops.gemm(a, b, acc, m, n, k, am, bm, flags=DS_EPI_ACCUM)
    assert_close(acc, (acc0 + Ar @ Br.T).cpu().double(), 1e-5, "gemm accumulate, wide blocks")


@pytest.mark.parametrize("am,bm,m,n,k", [
    (DS_K_MAJOR, DS_K_MAJOR, 1024, 1024, 4096),     # the BERT-48 layer's narrow input gradients
    (DS_K_MAJOR, DS_MN_MAJOR, 1024, 1024, 1024),    # its attention output projection
    (DS_K_MAJOR, DS_K_MAJOR, 200, 328, 2048),       # ragged edge tiles
    (DS_MN_MAJOR, DS_MN_MAJOR, 320, 192, 1152),     # 18 k-tiles
    (DS_MN_MAJOR, DS_K_MAJOR, 64, 64, 1024),        # one block
    (DS_K_MAJOR, DS_MN_MAJOR, 448, 1024, 3072),
])
def test_gemm_blocks_whose_waves_split_the_k_steps(am, bm, m, n, k):
    """64x64 blocks under a reduction of at least 16 (an even number of) k-tiles: each of the four waves multiplies the whole
    tile over one 16-deep k-step of every k-tile and the partial tiles meet in LDS.  All operand-major pairs, ragged edges,
    the vector epilogue's terms and the fp32 accumulate."""
    r = rng(m * 3 + n * 5 + k * 7 + am * 2 + bm)
    A = (r.standard_normal((m, k)) * 0.5).astype(np.float32)
    B = (r.standard_normal((n, k)) * 0.5).astype(np.float32)
    a = dev(A if am == DS_K_MAJOR else A.T, torch.bfloat16)
    b = dev(B if bm == DS_K_MAJOR else B.T, torch.bfloat16)
    bias = dev(r.standard_normal(n), torch.float32)
    res = dev(r.standard_normal((m, n)), torch.float32)
    Ar = (a if am == DS_K_MAJOR else a.T).float().cpu().double()
    Br = (b if bm == DS_K_MAJOR else b.T).float().cpu().double()
    prod = Ar @ Br.T
    c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    ops.gemm(a, b, c, m, n, k, am, bm, flags=DS_EPI_BIAS, bias=bias, alpha=0.125)
    assert_close(c, 0.125 * prod + bias.cpu().double(), TOL["bf16"], "gemm, k-step waves, bf16 output")
    c32 = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    ops.gemm(a, b, c32, m, n, k, am, bm, flags=DS_EPI_OUT_F32 | DS_EPI_RESIDUAL | DS_EPI_RESIDUAL_F32, residual=res)
    assert_close(c32, prod + res.cpu().double(), 1e-5, "gemm, k-step waves, fp32 output + fp32 residual")
    acc0 = dev(r.standard_normal((m, n)), torch.float32)
    acc = acc0.clone()
    ops.gemm(a, b, acc, m, n, k, am, bm, flags=DS_EPI_ACCUM)
    assert_close(acc, acc0.cpu().double() + prod, 1e-5, "gemm accumulate, k-step waves")


@pytest.mark.parametrize("dt,m,n,kseg,nseg,agap,bgap", [
    ("bf16", 1024, 2048, 512, 4, 3, 0),      # 8-wave tiles; A's segments 3 rows apart beyond their length, B's back to back
    ("bf16", 256, 192, 128, 3, 0, 5),        # 4-wave tiles
    ("bf16", 256, 192, 256, 4, 2, 1),        # 16 k-tiles under 64x64 blocks: the waves split the k-steps
    ("bf16", 4096, 1024, 1024, 8, 2, 1),     # a weight gradient over 8 micro-batches
    ("bf16", 1024, 1024, 1408, 2, -1, 0),    # A's segment stride 0: both segments read the same rows
    ("fp32", 512, 256, 96, 5, 1, 2),
])
def test_gemm_segmented_reduction(dt, m, n, kseg, nseg, agap, bgap):
    """ds_gemm_desc.k_segment: C += sum over segments s of A_s^T B_s with the segments' first rows a fixed stride apart (rows
    of other tensors in between, as in a stash whose slots hold one micro-batch each); against the sum of the per-segment
    products, through the plain launch, the accumulate epilogue and a grouped launch."""
    r = rng(m + n + kseg * nseg)
    tdt = DT[dt]
    arows = kseg + agap if agap >= 0 else 0          # rows from one segment's start to the next
    brows = kseg + bgap
    a = dev(r.standard_normal((max(arows, 1) * (nseg - 1) + kseg, m)) * 0.5, tdt)
    b = dev(r.standard_normal((brows * (nseg - 1) + kseg, n)) * 0.5, tdt)
    ref = torch.zeros(m, n, dtype=torch.float64)
    for s_ in range(nseg):
        As = a[s_ * arows: s_ * arows + kseg].float().cpu().double()
        Bs = b[s_ * brows: s_ * brows + kseg].float().cpu().double()
        ref += As.T @ Bs
    kw = dict(k_segment=kseg, a_segment_stride=arows * m, b_segment_stride=brows * n)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    ops.gemm(a, b, c, m, n, kseg * nseg, DS_MN_MAJOR, DS_MN_MAJOR, flags=DS_EPI_OUT_F32, **kw)
    assert_close(c, ref, 1e-5 if dt == "bf16" else 1e-5, "segmented reduction")
    acc0 = dev(r.standard_normal((m, n)), torch.float32)
    acc = acc0.clone()
    ops.gemm(a, b, acc, m, n, kseg * nseg, DS_MN_MAJOR, DS_MN_MAJOR, flags=DS_EPI_ACCUM, **kw)
    assert_close(acc, acc0.cpu().double() + ref, 1e-5, "segmented reduction, accumulate")
    if dt == "bf16":
        for cfg in (1, 3):
            g = acc0.clone()
            ops.gemm_grouped([dict(a=a, b=b, c=g, m=m, n=n, k=kseg * nseg, a_major=DS_MN_MAJOR, b_major=DS_MN_MAJOR, flags=DS_EPI_ACCUM,
                                   cfg=cfg, **kw)])
            assert_close(g, acc0.cpu().double() + ref, 1e-5, "segmented reduction, grouped launch cfg %d" % cfg)
    with pytest.raises((ValueError, RuntimeError)):
        ops.gemm(a, b, c, m, n, kseg * nseg, DS_MN_MAJOR, DS_MN_MAJOR, flags=DS_EPI_OUT_F32, k_segment=kseg + 8, a_segment_stride=0, b_segment_stride=0)


@pytest.mark.parametrize("am,bm", [(0, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(128, 256, 8192), (248, 120, 6144), (384, 128, 16384)])
def test_gemm_split_k_by_workspace(am, bm, m, n, k):
    """A few output tiles under a long reduction: with a workspace the library cuts k into slices; the result equals the
    unsplit product up to fp32 summation order, is the same bit for bit on every run, and the workspace comes back zeroed
    where the library counts arrivals."""
    r = rng(m + n + k)
    A = (r.standard_normal((m, k)) * 0.5).astype(np.float32)
    B = (r.standard_normal((n, k)) * 0.5).astype(np.float32)
    a = dev(A if am == DS_K_MAJOR else A.T, torch.bfloat16)
    b = dev(B if bm == DS_K_MAJOR else B.T, torch.bfloat16)
    bias = dev(r.standard_normal(n), torch.float32)
    ws = torch.zeros(ops.gemm_workspace_bytes(m, n), dtype=torch.uint8, device="cuda")
    outs = []
    for _ in range(3):
        c = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
        ops.gemm(a, b, c, m, n, k, am, bm, flags=DS_EPI_BIAS | DS_EPI_OUT_F32, bias=bias, workspace=ws)
        outs.append(c)
    plain = torch.empty_like(outs[0])
    ops.gemm(a, b, plain, m, n, k, am, bm, flags=DS_EPI_BIAS | DS_EPI_OUT_F32, bias=bias)
    Ar = (a if am == DS_K_MAJOR else a.T).cpu().double()
    Br = (b if bm == DS_K_MAJOR else b.T).cpu().double()
    assert_close(outs[0], Ar @ Br.T + bias.cpu().double(), 1e-5, "split-K gemm")
    assert_close(outs[0], plain, 1e-5, "split-K vs unsplit")
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    assert int(ws[:4096].count_nonzero()) == 0
    with pytest.raises(Exception):
        ops.gemm(a, b, outs[0], m, n, k, am, bm, flags=DS_EPI_OUT_F32, workspace=ws[:8192])   # too small


@pytest.mark.parametrize("dt", ["fp32", "bf16"])
def test_gemm_epilogues(dt):
    m, n, k = 192, 160, 96
    r = rng(5)
    x = dev(r.standard_normal((m, k)), DT[dt])
    w = dev(r.standard_normal((k, n)) * 0.2, DT[dt])
    bias = dev(r.standard_normal(n), torch.float32)
    res = dev(r.standard_normal((m, n)), DT[dt])
    ref = x.cpu().double() @ w.cpu().double() + bias.cpu().double()
    y = ops.dense(x, w, bias, residual=res)
    assert_close(y, ref + res.cpu().double(), TOL[dt], "bias+residual")
    pre, act = ops.dense(x, w, bias, gelu=True)
    assert_close(pre, ref, TOL[dt], "pre-gelu")
    assert_close(act, ob.gelu(ref), TOL[dt], "gelu")
    # relu
    c = torch.empty(m, n, dtype=DT[dt], device="cuda")
    ops.gemm(x, w, c, m, n, k, DS_K_MAJOR, DS_MN_MAJOR, flags=DS_EPI_BIAS | DS_EPI_RELU, bias=bias)
    assert_close(c, ref.clamp(min=0), TOL[dt], "relu")
    # dgelu: c = (x w) * gelu'(aux)
    aux = dev(r.standard_normal((m, n)), DT[dt])
    ops.gemm(x, w, c, m, n, k, DS_K_MAJOR, DS_MN_MAJOR, flags=DS_EPI_DGELU, c2=aux)
    a64 = aux.cpu().double().requires_grad_(True)
    (gp,) = torch.autograd.grad(ob.gelu(a64).sum(), a64)
    assert_close(c, (x.cpu().double() @ w.cpu().double()) * gp, TOL[dt], "dgelu")
    # gelu with its derivative kept for backward, then the multiply epilogue that consumes it
    from dapple_amd._lib import DS_EPI_GELU_GRAD, DS_EPI_MUL
    kept = torch.empty(m, n, dtype=DT[dt], device="cuda")
    act2 = torch.empty_like(kept)
    ops.gemm(x, w, kept, m, n, k, DS_K_MAJOR, DS_MN_MAJOR, flags=DS_EPI_BIAS | DS_EPI_GELU | DS_EPI_GELU_GRAD, bias=bias, c2=act2)
    r64 = ref.clone().requires_grad_(True)
    (gref,) = torch.autograd.grad(ob.gelu(r64).sum(), r64)
    assert_close(act2, ob.gelu(ref), TOL[dt], "gelu (derivative kept)")
    assert_close(kept, gref, TOL[dt], "kept gelu derivative")
    ops.gemm(x, w, c, m, n, k, DS_K_MAJOR, DS_MN_MAJOR, flags=DS_EPI_MUL, c2=aux)
    assert_close(c, (x.cpu().double() @ w.cpu().double()) * aux.cpu().double(), TOL[dt], "multiply epilogue")
    # fp32 output and accumulate (wgrad form: both operands MN-major), twice -> 2x + initial
    acc0 = r.standard_normal((k, n)).astype(np.float32)
    acc = dev(acc0)
    dy = dev(r.standard_normal((m, n)), DT[dt])
    for _ in range(2):
        ops.gemm(x, dy, acc, k, n, m, DS_MN_MAJOR, DS_MN_MAJOR, lda=k, ldb=n, ldc=n, flags=DS_EPI_ACCUM)
    assert_close(acc, torch.from_numpy(acc0).double() + 2 * (x.cpu().double().T @ dy.cpu().double()), 1e-5, "accum")
    out32 = torch.empty(m, n, dtype=torch.float32, device="cuda")
    ops.gemm(x, w, out32, m, n, k, DS_K_MAJOR, DS_MN_MAJOR, flags=DS_EPI_OUT_F32, alpha=0.5)
    assert_close(out32, 0.5 * (x.cpu().double() @ w.cpu().double()), 1e-5, "out_f32 alpha")


@pytest.mark.parametrize("m,n,k", [(192, 160, 96), (1024, 1024, 1024), (1024, 3072, 512)])
def test_gemm_adds_into_an_fp32_residual_stream(m, n, k):
    """bf16 operands, fp32 residual in (DS_EPI_RESIDUAL_F32), the sum kept in fp32 (DS_EPI_OUT_F32) or rounded to bf16."""
    from dapple_amd._lib import DS_EPI_RESIDUAL_F32
    r = rng(m + n + k)
    x = dev(r.standard_normal((m, k)), torch.bfloat16)
    w = dev(r.standard_normal((k, n)) * 0.1, torch.bfloat16)
    bias = dev(r.standard_normal(n), torch.float32)
    res = dev(r.standard_normal((m, n)) * 3, torch.float32)
    ref = x.cpu().double() @ w.cpu().double() + bias.cpu().double() + res.cpu().double()
    c32 = torch.empty(m, n, dtype=torch.float32, device="cuda")
    ops.gemm(x, w, c32, m, n, k, DS_K_MAJOR, DS_MN_MAJOR, flags=DS_EPI_BIAS | DS_EPI_RESIDUAL | DS_EPI_RESIDUAL_F32 | DS_EPI_OUT_F32,
             bias=bias, residual=res)
    assert_close(c32, ref, 1e-5, "fp32 sum")
    c16 = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    ops.gemm(x, w, c16, m, n, k, DS_K_MAJOR, DS_MN_MAJOR, flags=DS_EPI_BIAS | DS_EPI_RESIDUAL | DS_EPI_RESIDUAL_F32, bias=bias, residual=res)
    assert torch.equal(c16, c32.to(torch.bfloat16))


@pytest.mark.parametrize("dt", ["fp32", "bf16"])
def test_gemm_batched_head_views(dt):
    B, N, S, D = 2, 4, 32, 16
    H = N * D
    r = rng(9)
    qkv = dev(r.standard_normal((B * S, 3 * H)), DT[dt])
    scores = torch.empty(B, N, S, S, dtype=torch.float32, device="cuda")
    kview = qkv.view(-1)[H:]
    ops.gemm(qkv, kview, scores, S, S, D, DS_K_MAJOR, DS_K_MAJOR, lda=3 * H, ldb=3 * H, ldc=S, flags=DS_EPI_OUT_F32,
             batch=B * N, batch_inner=N, a_strides=(S * 3 * H, D), b_strides=(S * 3 * H, D), c_strides=(N * S * S, S * S))
    q = qkv[:, :H].cpu().double().reshape(B, S, N, D).permute(0, 2, 1, 3)
    k = qkv[:, H:2 * H].cpu().double().reshape(B, S, N, D).permute(0, 2, 1, 3)
    assert_close(scores, q @ k.transpose(-1, -2), 1e-5, "scores")


@pytest.mark.parametrize("B,N,Q,K", [(1, 16, 512, 896), (2, 3, 64, 192), (1, 1, 128, 64)])
def test_gemm_head_scores_fp32_out(B, N, Q, K):
    # bf16, both operands K-major, reduction of exactly 64, fp32 output: the per-head score products (own kernel)
    D = 64
    H = N * D
    r = rng(Q + K + N)
    q = dev(r.standard_normal((Q, B, H)), torch.bfloat16)           # [i][b][n*D], as the XLNet stage holds q
    kv = dev(r.standard_normal((K, B, 2 * H)), torch.bfloat16)      # [j][b][k | v]
    out = torch.full((B, N, Q, K), float("nan"), dtype=torch.float32, device="cuda")
    ops.gemm(q, kv, out, Q, K, D, DS_K_MAJOR, DS_K_MAJOR, lda=B * H, ldb=B * 2 * H, ldc=K, flags=DS_EPI_OUT_F32, alpha=0.25,
             batch=B * N, batch_inner=N, a_strides=(H, D), b_strides=(2 * H, D), c_strides=(N * Q * K, Q * K))
    qh = q.cpu().double().reshape(Q, B, N, D).permute(1, 2, 0, 3)
    kh = kv[:, :, :H].cpu().double().reshape(K, B, N, D).permute(1, 2, 0, 3)
    assert_close(out, 0.25 * (qh @ kh.transpose(-1, -2)), 1e-5, "head scores")


@pytest.mark.parametrize("dt", ["fp32", "bf16"])
@pytest.mark.parametrize("rows,cols", [(7, 64), (256, 1024), (33, 512), (5, 2048)])
def test_layernorm_fwd_bwd(dt, rows, cols):
    r = rng(rows + cols)
    x = dev(r.standard_normal((rows, cols)) * 2 + 0.5, DT[dt])
    g = dev(1 + 0.2 * r.standard_normal(cols), torch.float32)
    b = dev(0.3 * r.standard_normal(cols), torch.float32)
    dy = dev(r.standard_normal((rows, cols)), DT[dt])
    add = dev(r.standard_normal((rows, cols)), DT[dt])
    y, stats = ops.layernorm_fwd(x, g, b, 1e-12)
    x64 = x.cpu().double().requires_grad_(True)
    g64 = g.cpu().double().requires_grad_(True)
    b64 = b.cpu().double().requires_grad_(True)
    ref = ob.layer_norm(x64, g64, b64)
    tol = 1e-5 if dt == "fp32" else 1e-2
    assert_close(y, ref, tol, "ln fwd")
    dx_ref, dg_ref, db_ref = torch.autograd.grad(ref, [x64, g64, b64], dy.cpu().double())
    dg = torch.ones(cols, device="cuda")
    db = torch.ones(cols, device="cuda")
    dcs = torch.ones(cols, device="cuda")
    dx = ops.layernorm_bwd(dy, x, g, stats, dg, db, dcs, dx_add=add)
    assert_close(dx, dx_ref + add.cpu().double(), tol, "ln dx")
    assert_close(dg, dg_ref + 1, 1e-4, "ln dgamma (accumulates)")
    assert_close(db, db_ref + 1, 1e-4, "ln dbeta")
    assert_close(dcs, dx_ref.sum(0) + 1, 1e-4 if dt == "fp32" else 1e-2, "ln colsum")
    # the same pass in two calls: dx alone, then the parameter gradients (and the column sums of that dx)
    dx2 = ops.layernorm_bwd(dy, x, g, stats, None, None, None, dx_add=None)
    assert_close(dx2, dx_ref, tol, "ln dx (rows only)")
    dg2, db2, dcs2 = torch.ones(cols, device="cuda"), torch.ones(cols, device="cuda"), torch.ones(cols, device="cuda")
    ops.layernorm_param_grads(dy, x, stats, dg2, db2, dx=dx2, d_colsum=dcs2)
    assert_close(dg2, dg_ref + 1, 1e-4, "ln dgamma (separate call)")
    assert_close(db2, db_ref + 1, 1e-4, "ln dbeta (separate call)")
    assert_close(dcs2, dx2.double().cpu().sum(0) + 1, 1e-4, "ln colsum (separate call)")
    dg3, db3 = torch.zeros(cols, device="cuda"), torch.zeros(cols, device="cuda")
    ops.layernorm_param_grads(dy, x, stats, dg3, db3)
    assert_close(dg3, dg_ref, 1e-4, "ln dgamma (no colsum)")


@pytest.mark.parametrize("rows,cols", [(7, 64), (1024, 1024), (33, 520), (5, 2048)])
def test_layernorm_on_an_fp32_stream(rows, cols):
    """The kernels of a bf16 stage with an fp32 residual stream: fp32 in, the bf16 operand copy and the fp32 carrier out;
    both against torch's layer_norm and its autograd in fp64 (the fp32 outputs at 1e-5, their bf16 copies at rounding)."""
    r = rng(rows + cols)
    x = dev(r.standard_normal((rows, cols)) * 1.5 + 0.3, torch.float32)
    gamma = dev(1 + 0.1 * r.standard_normal(cols), torch.float32)
    beta = dev(0.1 * r.standard_normal(cols), torch.float32)
    dy = dev(r.standard_normal((rows, cols)), torch.float32)
    y16, y32, stats = ops.layernorm_fwd_mixed(x, gamma, beta, 1e-12)
    x64 = x.cpu().double().requires_grad_(True)
    g64, b64 = gamma.cpu().double().requires_grad_(True), beta.cpu().double().requires_grad_(True)
    ref = torch.nn.functional.layer_norm(x64, (cols,), g64, b64, 1e-12)
    assert_close(y32, ref.detach(), 1e-5, "y fp32")
    assert torch.equal(y16, y32.to(torch.bfloat16))
    assert ops.layernorm_fwd_mixed(x, gamma, beta, 1e-12, want_f32=False)[1] is None
    dxr, dgr, dbr = torch.autograd.grad(ref, [x64, g64, b64], dy.cpu().double())
    dg = torch.full((cols,), 2.0, device="cuda")
    db = torch.full((cols,), -1.0, device="cuda")
    dcs = torch.zeros(cols, device="cuda")
    dx16, dx32 = ops.layernorm_bwd_mixed(dy, x, gamma, stats, dg, db, dcs)
    assert_close(dx32, dxr, 1e-5, "dx fp32")
    assert torch.equal(dx16, dx32.to(torch.bfloat16))
    assert_close(dg - 2.0, dgr, 1e-5, "d_gamma (added to)")
    assert_close(db + 1.0, dbr, 1e-5, "d_beta (added to)")
    assert_close(dcs, dxr.sum(0), 1e-4, "column sums of dx", floor=float(dxr.abs().max()) * rows ** 0.5)
    # the split form: dx alone (bit-identical to the fused kernel's), then the parameter gradients from the bf16 copy of dy
    ex16, ex32, dy16 = ops.layernorm_bwd_mixed(dy, x, gamma, stats, want_dy_bf16=True)
    assert torch.equal(dy16, dy.to(torch.bfloat16))
    assert_close(ex32, dxr, 1e-5, "dx fp32, rows only")
    assert torch.equal(ex16, ex32.to(torch.bfloat16))
    assert ops.layernorm_bwd_mixed(dy, x, gamma, stats, want_f32=False)[1] is None
    dg2 = torch.full((cols,), 2.0, device="cuda")
    db2 = torch.full((cols,), -1.0, device="cuda")
    dcs2 = torch.zeros(cols, device="cuda")
    ops.layernorm_param_grads_mixed(dy16, x, stats, dg2, db2, ex16, dcs2)
    # against the same sums taken over the rounded copies in fp64: what the kernel is asked to compute
    xh = (x64.detach() - x64.detach().mean(1, keepdim=True)) / torch.sqrt(x64.detach().var(1, unbiased=False, keepdim=True) + 1e-12)
    d16 = dy16.cpu().double()
    assert_close(dg2 - 2.0, (d16 * xh).sum(0), 1e-5, "d_gamma from the bf16 copy", floor=float(d16.abs().max()) * rows ** 0.5)
    assert_close(db2 + 1.0, d16.sum(0), 1e-5, "d_beta from the bf16 copy", floor=float(d16.abs().max()) * rows ** 0.5)
    assert_close(dcs2, ex16.cpu().double().sum(0), 1e-5, "column sums of the bf16 dx", floor=float(dxr.abs().max()) * rows ** 0.5)
    # and within bf16 rounding of the exact gradients
    assert_close(dg2 - 2.0, dgr, 2e-2, "d_gamma, deferred", floor=float(dgr.abs().max()))
    assert_close(db2 + 1.0, dbr, 2e-2, "d_beta, deferred", floor=float(dbr.abs().max()))
    dg3 = torch.zeros(cols, device="cuda"); db3 = torch.zeros(cols, device="cuda")
    ops.layernorm_param_grads_mixed(dy16, x, stats, dg3, db3)     # without the column sums
    assert torch.allclose(dg3, dg2 - 2.0, atol=1e-4 * float(dg3.abs().max())) and torch.allclose(db3, db2 + 1.0, atol=1e-4 * float(db3.abs().max()))
    # the split form that rounds nothing on the way: fp32 copy of dy + the two per-row means, then the exact sums
    fx16, fx32, dyc, row_sums = ops.layernorm_bwd_mixed_rows(dy, x, gamma, stats)
    assert torch.equal(fx16, ex16) and torch.equal(fx32, ex32) and torch.equal(dyc, dy)
    dg4 = torch.full((cols,), 2.0, device="cuda")
    db4 = torch.full((cols,), -1.0, device="cuda")
    dcs4 = torch.zeros(cols, device="cuda")
    ops.layernorm_param_grads_exact(dyc, x, gamma, stats, row_sums, dg4, db4, dcs4)
    assert_close(dg4 - 2.0, dgr, 1e-5, "d_gamma, exact hand-over")
    assert_close(db4 + 1.0, dbr, 1e-5, "d_beta, exact hand-over")
    assert_close(dcs4, dxr.sum(0), 1e-4, "column sums of dx, exact hand-over", floor=float(dxr.abs().max()) * rows ** 0.5)


@pytest.mark.parametrize("dt", ["fp32", "bf16"])
@pytest.mark.parametrize("k", [16, 128, 512, 896])
def test_softmax_fwd_bwd(dt, k):
    B, N, Q = 2, 3, 5
    r = rng(k)
    s = dev(r.standard_normal((B, N, Q, k)) * 3, torch.float32)
    mask = dev((r.random((B, k)) > 0.3), torch.float32)
    scale = 0.125
    p = ops.softmax_fwd(s, scale, mask, -10000.0, DT[dt])
    s64 = (s.cpu().double() * scale + (1 - mask.cpu().double())[:, None, None, :] * -10000.0).requires_grad_(True)
    ref = torch.softmax(s64, -1)
    tol = 1e-5 if dt == "fp32" else 1e-2
    assert_close(p, ref, tol, "softmax")
    assert (p.float().sum(-1) - 1).abs().max().item() < (1e-5 if dt == "fp32" else 2e-2)
    p0 = ops.softmax_fwd(s, scale, None, 0.0, DT[dt])
    assert_close(p0, torch.softmax(s.cpu().double() * scale, -1), tol, "softmax no mask")
    dp = dev(r.standard_normal((B, N, Q, k)), torch.float32)
    ds = ops.softmax_bwd(p, dp, scale)
    pr = p.cpu().double()
    want = scale * pr * (dp.cpu().double() - (dp.cpu().double() * pr).sum(-1, keepdim=True))
    assert_close(ds, want, tol, "softmax bwd")


@pytest.mark.parametrize("dt", ["fp32", "bf16"])
def test_colsum(dt):
    x = dev(rng(4).standard_normal((1000, 200)), DT[dt])
    out = torch.ones(200, device="cuda")
    ops.colsum_accum(x, out)
    assert_close(out, x.cpu().double().sum(0) + 1, 1e-5, "colsum")
    # narrow matrices (several rows per wave-wide read), a row count that is not a multiple of that, many rows
    for rows, cols in ((1003, 64), (7, 32), (200001, 64), (4099, 8), (33, 128)):
        x = dev(rng(rows + cols).standard_normal((rows, cols)), DT[dt])
        out = torch.ones(cols, device="cuda")
        ops.colsum_accum(x, out)
        assert_close(out, x.cpu().double().sum(0) + 1, 1e-4, "colsum %dx%d" % (rows, cols))


@pytest.mark.parametrize("B,N,S,use_mask,spread", [
    (1, 1, 64, False, 0.7), (2, 3, 128, True, 0.7), (2, 16, 512, True, 0.7), (1, 2, 1024, False, 0.7),
    (1, 2, 192, True, 0.7), (2, 1, 320, True, 0.7), (1, 1, 2048, True, 0.7),   # ragged last tile; the maximum
    (2, 16, 512, False, 0.7), (1, 3, 320, False, 2.5), (2, 2, 1024, False, 4.0)])
def test_fused_attention_fwd_bwd(B, N, S, use_mask, spread):
    # spread 2.5 / 4.0: scores with a standard deviation of 6 / 16, so that the running maximum of the mask-free kernels,
    # which only moves when a step exceeds it by a factor 2^8, does move in later steps for some rows and not for others
    D, H = 64, N * 64
    r = rng(S + N)
    qkv = dev(r.standard_normal((B * S, 3 * H)) * np.array([spread] * (2 * H) + [0.7] * H), torch.bfloat16)
    dctx = dev(r.standard_normal((B * S, H)), torch.bfloat16)
    mask = None
    if use_mask:
        m = (r.random((B, S)) > 0.2).astype(np.float32)
        m[:, 0] = 1
        mask = dev(m)
    scale = 1.0 / math.sqrt(D)
    ctx, lse = ops.attention_fwd(qkv, B, N, S, scale, mask)
    x = qkv.cpu().double().requires_grad_(True)
    q, k, v = (x[:, i * H:(i + 1) * H].reshape(B, S, N, D).permute(0, 2, 1, 3) for i in range(3))
    sc = q @ k.transpose(-1, -2) * scale
    if use_mask:
        sc = sc + (1.0 - mask.cpu().double())[:, None, None, :] * -10000.0
    ref = (torch.softmax(sc, -1) @ v).permute(0, 2, 1, 3).reshape(B * S, H)
    assert_close(ctx, ref, 1e-2, "fused attention fwd")
    assert_close(lse, torch.logsumexp(sc, -1), 1e-3, "logsumexp")
    (dx,) = torch.autograd.grad(ref, x, dctx.cpu().double())
    dqkv = ops.attention_bwd(qkv, ctx, lse, dctx, B, N, S, scale, mask)
    for i, name in enumerate(("dq", "dk", "dv")):
        assert_close(dqkv[:, i * H:(i + 1) * H], dx[:, i * H:(i + 1) * H], 2e-2, "fused attention " + name)


def test_fused_attention_with_a_negative_scale():
    """The mask-free short form of the steps takes the maximum of the raw scores, which is the maximum of the scaled ones
    only for a positive scale: any other scale must take the general form and still be right."""
    B, N, S, D = 1, 2, 128, 64
    H = N * D
    r = rng(17)
    qkv = dev(r.standard_normal((B * S, 3 * H)) * 0.7, torch.bfloat16)
    dctx = dev(r.standard_normal((B * S, H)), torch.bfloat16)
    scale = -0.2
    ctx, lse = ops.attention_fwd(qkv, B, N, S, scale)
    x = qkv.cpu().double().requires_grad_(True)
    q, k, v = (x[:, i * H:(i + 1) * H].reshape(B, S, N, D).permute(0, 2, 1, 3) for i in range(3))
    sc = q @ k.transpose(-1, -2) * scale
    ref = (torch.softmax(sc, -1) @ v).permute(0, 2, 1, 3).reshape(B * S, H)
    assert_close(ctx, ref, 1e-2, "fused attention fwd, negative scale")
    assert_close(lse, torch.logsumexp(sc, -1), 1e-3, "logsumexp, negative scale")
    (dx,) = torch.autograd.grad(ref, x, dctx.cpu().double())
    dqkv = ops.attention_bwd(qkv, ctx, lse, dctx, B, N, S, scale)
    for i, name in enumerate(("dq", "dk", "dv")):
        assert_close(dqkv[:, i * H:(i + 1) * H], dx[:, i * H:(i + 1) * H], 2e-2, "fused attention %s, negative scale" % name)


def test_fused_attention_backward_with_keys_that_share_a_common_part():
    """Keys = a large common vector + small differences (what a deep, randomly initialised stack drives its token vectors
    to): dq = dS k is then a small difference of large terms.  The plain kernel's dq carries the row sums of the
    bf16-rounded dS times the common part; ds_attention_bwd_centered takes that out: its dq meets the 2e-2 bar of its own
    scale where the plain kernel misses it by a wide margin.  dk and dv are untouched."""
    B, N, S, D = 2, 4, 256, 64
    H = N * D
    r = rng(91)
    common = r.standard_normal((1, 3 * H)) * np.concatenate([np.zeros(H), np.full(H, 4.0), np.zeros(H)])
    qkv = dev(r.standard_normal((B * S, 3 * H)) * 0.5 + common, torch.bfloat16)
    dctx = dev(r.standard_normal((B * S, H)), torch.bfloat16)
    scale = 1.0 / math.sqrt(D)
    ctx, lse = ops.attention_fwd(qkv, B, N, S, scale)
    x = qkv.cpu().double().requires_grad_(True)
    q, k, v = (x[:, i * H:(i + 1) * H].reshape(B, S, N, D).permute(0, 2, 1, 3) for i in range(3))
    ref = (torch.softmax(q @ k.transpose(-1, -2) * scale, -1) @ v).permute(0, 2, 1, 3).reshape(B * S, H)
    (dx,) = torch.autograd.grad(ref, x, dctx.cpu().double())
    kmean = ops.attention_key_mean(qkv, B, N, S)
    want_mean = qkv[:, H:2 * H].float().reshape(B, S, H).mean(1)
    assert_close(kmean, want_mean, 1e-5, "key mean")
    plain = ops.attention_bwd(qkv, ctx, lse, dctx, B, N, S, scale)
    centred = ops.attention_bwd(qkv, ctx, lse, dctx, B, N, S, scale, key_mean=kmean)
    err_plain = rel_err(plain[:, :H], dx[:, :H])[1]
    err_centred = rel_err(centred[:, :H], dx[:, :H])[1]
    print("dq rel l2: plain %.3e, centred %.3e" % (err_plain, err_centred))
    assert err_centred <= 2e-2 and err_plain > 3 * err_centred
    assert torch.equal(plain[:, H:], centred[:, H:])
    for i, name in ((1, "dk"), (2, "dv")):
        assert_close(centred[:, i * H:(i + 1) * H], dx[:, i * H:(i + 1) * H], 2e-2, "fused attention " + name)


def test_fused_attention_rejects_other_shapes():
    qkv = torch.zeros(64, 3 * 32, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="head size"):
        ops.attention_fwd(qkv, 1, 1, 64, 1.0)
    with pytest.raises(ValueError, match="multiple of 64"):
        ops.attention_fwd(torch.zeros(48, 192, dtype=torch.bfloat16, device="cuda"), 1, 1, 48, 1.0)


def test_layernorm_widest_row_and_single_row():
    """The widest row the kernel takes (64 lanes x 8 vectors x 8 bf16 = 4096 columns), and a single row."""
    for rows, cols in ((3, 4096), (1, 1024)):
        r = rng(rows * 7 + cols)
        x = dev(r.standard_normal((rows, cols)), torch.bfloat16)
        g = dev(1 + 0.2 * r.standard_normal(cols), torch.float32)
        b = dev(0.3 * r.standard_normal(cols), torch.float32)
        dy = dev(r.standard_normal((rows, cols)), torch.bfloat16)
        y, stats = ops.layernorm_fwd(x, g, b, 1e-12)
        x64 = x.cpu().double().requires_grad_(True)
        g64, b64 = g.cpu().double().requires_grad_(True), b.cpu().double().requires_grad_(True)
        ref = ob.layer_norm(x64, g64, b64)
        assert_close(y, ref, 1e-2, "ln fwd")
        dx_ref, dg_ref, db_ref = torch.autograd.grad(ref, [x64, g64, b64], dy.cpu().double())
        dg, db = torch.zeros(cols, device="cuda"), torch.zeros(cols, device="cuda")
        dx = ops.layernorm_bwd(dy, x, g, stats, dg, db, None)
        assert_close(dx, dx_ref, 1e-2, "ln dx")
        assert_close(dg, dg_ref, 1e-4, "ln dgamma")
        assert_close(db, db_ref, 1e-4, "ln dbeta")
    with pytest.raises(ValueError):
        ops.layernorm_fwd(torch.zeros(2, 4104, dtype=torch.bfloat16, device="cuda"), torch.ones(4104, device="cuda"),
                          torch.zeros(4104, device="cuda"), 1e-12)
