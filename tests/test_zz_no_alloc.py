"""ds_gemm_static_scratch - the entry point that allocates nothing - against ds_gemm with a caller workspace."""
import numpy as np
import pytest
import torch

from dapple_amd import ops
from dapple_amd._lib import DS_EPI_BIAS, DS_EPI_OUT_F32, DS_EPI_RESIDUAL, DS_K_MAJOR, DS_MN_MAJOR
from util import dev

pytestmark = pytest.mark.gpu


def _case(seed, m, n, k, am, bm):
    r = np.random.Generator(np.random.PCG64(seed))
    A = (r.standard_normal((m, k)) * 0.5).astype(np.float32)
    B = (r.standard_normal((n, k)) * 0.5).astype(np.float32)
    a = dev(A if am == DS_K_MAJOR else A.T, torch.bfloat16)
    b = dev(B if bm == DS_K_MAJOR else B.T, torch.bfloat16)
    bias = dev(r.standard_normal(n), torch.float32)
    res = dev(r.standard_normal((m, n)), torch.bfloat16)
    return a, b, bias, res


def test_static_scratch_gemm_equals_workspace_gemm_on_two_calls_in_a_row():
    """Two calls back to back through the C ABI, the second on a smaller problem that reuses the front of the scratch the
    first one filled: both equal ds_gemm with a caller workspace bit for bit (same kernel, same slices, same order of
    the fixed-order reduction), and the product itself is right."""
    from dapple_amd import _lib
    _lib.check(_lib.load().ds_gemm_static_scratch_init(), "ds_gemm_static_scratch_init")
    for seed, (m, n, k, am, bm) in enumerate([(512, 512, 8192, DS_K_MAJOR, DS_MN_MAJOR), (128, 256, 8192, DS_K_MAJOR, DS_K_MAJOR)]):
        a, b, bias, res = _case(70 + seed, m, n, k, am, bm)
        ws = torch.zeros(ops.gemm_workspace_bytes(m, n), dtype=torch.uint8, device="cuda")
        want = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        ops.gemm(a, b, want, m, n, k, am, bm, flags=DS_EPI_BIAS | DS_EPI_RESIDUAL, bias=bias, residual=res, workspace=ws)
        got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        ops.gemm(a, b, got, m, n, k, am, bm, flags=DS_EPI_BIAS | DS_EPI_RESIDUAL, bias=bias, residual=res, static_scratch=True)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "call %d changed the free device memory" % seed
        assert torch.equal(got, want), "call %d" % seed
        Ar = (a if am == DS_K_MAJOR else a.T).float()
        Br = (b if bm == DS_K_MAJOR else b.T).float()
        ref = Ar @ Br.T + bias + res.float()
        err = (got.float() - ref).abs().max().item() / ref.abs().max().item()
        assert err < 1e-2, "call %d: rel err %.3e against the fp32 product" % (seed, err)   # bf16 output rounding


def test_static_scratch_gemm_rejects_what_it_cannot_hold():
    a, b, bias, res = _case(80, 1024, 1024, 8192, DS_K_MAJOR, DS_MN_MAJOR)
    c = torch.empty(1024, 1024, dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError, match="scratch holds 16"):
        ops.gemm(a, b, c, 1024, 1024, 8192, flags=DS_EPI_OUT_F32, static_scratch=True)
    a2, b2, _, _ = _case(81, 128, 128, 256, DS_K_MAJOR, DS_MN_MAJOR)
    c2 = torch.empty(128, 128, dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError, match="not a shape that is cut"):          # a reduction of 4 k-tiles is not sliced
        ops.gemm(a2, b2, c2, 128, 128, 256, flags=DS_EPI_OUT_F32, static_scratch=True)
    f2 = torch.empty(128, 256, dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError, match="bf16"):
        ops.gemm(f2, f2.T.contiguous(), c2, 128, 128, 256, flags=0, static_scratch=True)
