"""bench.py's roofline.traffic comes from the counter summary committed under profiles/: the rows parse, cover every GEMM
shape of the headline workload's layer, and name the kernel the library sends that shape to today (otherwise the counters
have to be taken again)."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(__file__), ".."))
import bench            # noqa: E402
import bench_calib      # noqa: E402


def test_traffic_rows_parse_and_cover_the_layer():
    rows = bench.traffic_rows()
    shapes = {(r[1].split(" (")[0], r[2]) for r in rows}
    for name, m, n, k, am, bm, acc in bench_calib.layer_shapes():
        assert (name, (m, n, k)) in shapes, name
    for tag, name, (m, n, k), rd, wr, alg in rows:
        acc = "C +=" in name
        assert alg == 2 * (m * k + n * k) + (8 if acc else 2) * m * n
        assert wr >= (4 if acc else 2) * m * n and rd >= 2 * (m * k + n * k)      # nothing moves less than the operands once
    dom = bench.traffic_of("gemm_ks4_kernel<bf16,64,64,K,K>", "bert48_half", 4)
    assert dom is not None and 30e6 < dom < 45e6
    assert bench.traffic_of("gemm_ks4_kernel<bf16,64,64,K,K>", "xlnet36_half", 4) is None
    assert bench.traffic_of("gemm8_kernel<bf16,128,128,MN,MN>", "bert48_half", 3) is None   # grouping without a counter run


@pytest.mark.gpu
def test_rows_name_the_kernel_each_shape_runs_on():
    from dapple_amd import _lib, ops
    from dapple_amd._lib import DS_EPI_ACCUM, DS_K_MAJOR
    rows = {(r[1].split(" (")[0], r[2]): r[0] for r in bench.traffic_rows()}
    bf = torch.bfloat16
    for name, m, n, k, am, bm, acc in bench_calib.layer_shapes():
        a = torch.zeros((m, k) if am == DS_K_MAJOR else (k, m), device="cuda", dtype=bf)
        b = torch.zeros((n, k) if bm == DS_K_MAJOR else (k, n), device="cuda", dtype=bf)
        c = torch.zeros(m, n, device="cuda", dtype=torch.float32 if acc else bf)
        _lib.profile(True)
        _lib.profile_dump()
        ops.gemm(a, b, c, m, n, k, am, bm, flags=DS_EPI_ACCUM if acc else 0)
        torch.cuda.synchronize()
        tags = list(_lib.profile_dump())
        _lib.profile(False)
        assert tags == [rows[(name, (m, n, k))]], "%s: runs on %s, counters were taken on %s" % (name, tags, rows[(name, (m, n, k))])
