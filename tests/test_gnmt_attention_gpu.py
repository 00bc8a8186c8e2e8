"""Decoder cell 0 under the attention wrapper (GNMT's first device, behind the encoder) through the C ABI against the
fp64 CPU oracle (fp32: 1e-4)."""
import numpy as np
import pytest
import torch

from dapple_amd import runtime, synthetic
from oracle import gnmt as og
from util import assert_close, dev

pytestmark = pytest.mark.gpu
TOL = 1e-4
ORDER = [og.EMB_DEC, og.ATT_CELL + "/kernel", og.ATT_CELL + "/bias", og.ATT_MEM, og.ATT_Q, og.ATT_V, og.ATT_G, og.ATT_B]


def oracle_weights(w_np):
    w = {k: torch.tensor(v, dtype=torch.float64) for k, v in w_np.items()}
    w[og.ATT_G] = w[og.ATT_G].reshape(())
    return {k: v.requires_grad_(True) for k, v in w.items()}


def run_case(U, V, B, T, S, M, K=1, seed=0, init=0.3, lengths=True, overlap=False, tol=TOL):
    w_np = synthetic.gnmt_attention_weights(synthetic.SEED_WEIGHT + seed, U, V, init_weight=init, perturb=True)
    r = np.random.Generator(np.random.PCG64(700 + seed))
    ids_np = [r.integers(0, V, (B, T)).astype(np.int32) for _ in range(M)]
    mem_np = [r.standard_normal((S, B, U)).astype(np.float32) for _ in range(M)]
    dys_np = synthetic.upstream_grads(synthetic.SEED_GRAD + seed, M, (T, B, U))
    len_np = [r.integers(1, S + 1, B).astype(np.int32) if lengths else None for _ in range(M)]
    if lengths:
        len_np[0][0] = S; len_np[0][-1] = 1
    st = runtime.gnmt_attention_stage(U, V, B, T, S, stash_slots=K)
    assert st.weight_names == ORDER
    st.bind(w_np)
    if overlap:
        st.enable_overlap()
    ids, mems, dys = [dev(i) for i in ids_np], [dev(m) for m in mem_np], [dev(d) for d in dys_np]
    lens = [None if l is None else dev(l) for l in len_np]
    outs = [torch.empty(T, B, U, device="cuda") for _ in range(M)]
    atts = [torch.empty(T, B, U, device="cuda") for _ in range(M)]
    dmems = [torch.empty(S, B, U, device="cuda") for _ in range(M)]
    runtime.StageRuntime(st, 0, K, M).step(mems, dys, outs, dmems,
                                           before_forward=lambda slot, j: st.set_decoder_inputs(slot, ids[j], lens[j], atts[j]))
    st.sync()
    wt = oracle_weights(w_np)
    acc = None
    for j in range(M):
        mo = torch.tensor(mem_np[j], dtype=torch.float64, requires_grad=True)
        lo = torch.full((B,), S) if len_np[j] is None else torch.tensor(len_np[j])
        out, att = og.attention_cell_forward(torch.tensor(ids_np[j]), mo, lo, wt)
        ps = [mo] + [wt[n] for n in ORDER]
        gs = torch.autograd.grad(out, ps, grad_outputs=torch.tensor(dys_np[j], dtype=torch.float64), allow_unused=True)
        gs = [torch.zeros_like(p) if g is None else g for g, p in zip(gs, ps)]   # a single step never reads its attention
        assert_close(outs[j], out.detach(), tol, "cell outputs mb%d" % j)
        assert_close(atts[j], att.detach(), tol, "attention mb%d" % j)
        assert_close(dmems[j], gs[0], tol, "memory grad mb%d" % j)
        if len_np[j] is not None:
            for b in range(B):
                if len_np[j][b] < S:
                    assert float(dmems[j][len_np[j][b]:, b].abs().max()) == 0.0     # nothing flows into the padded source steps
        acc = list(gs[1:]) if acc is None else [a + g for a, g in zip(acc, gs[1:])]
    big = max(float(g.abs().max()) for g in acc)
    for n, g in zip(ORDER, acc):
        assert_close(st.grads[n], g.reshape(st.grads[n].shape), tol, "accumulated grad " + n, floor=big)
    st.close()


def test_small_ragged_sources():
    run_case(U=32, V=40, B=4, T=5, S=7, M=3, K=2)


def test_full_length_sources_single_step():
    run_case(U=16, V=10, B=4, T=1, S=3, M=2, seed=1, lengths=False)


def test_repeated_target_ids_and_one_source_step():
    run_case(U=16, V=2, B=8, T=4, S=1, M=1, seed=2)


def test_overlapped_streams():
    run_case(U=32, V=40, B=4, T=4, S=6, M=4, K=2, seed=3, overlap=True)


def test_reference_shape_short():
    # units 1024, batch 64, 50 source steps (BASELINE configs[2]'s shape), 8 target steps
    run_case(U=1024, V=32000, B=64, T=8, S=50, M=1, seed=4, init=0.05)


def test_chain_encoder_attention_cell_decoder_cells():
    # device 0: encoder -> attention cell; device 1: decoder cells fed the first device's outputs (and, here, its attention)
    L, U, V, B, T, S = 2, 16, 20, 4, 3, 5
    ew = synthetic.gnmt_weights(81, L, U, V, init_weight=0.4, perturb=True)
    aw = synthetic.gnmt_attention_weights(82, U, V, init_weight=0.4, perturb=True)
    dw = synthetic.gnmt_decoder_weights(83, 1, 2, U, init_weight=0.4, perturb=True)
    r = np.random.Generator(np.random.PCG64(84))
    src, tgt = r.integers(0, V, (B, S)).astype(np.int32), r.integers(0, V, (B, T)).astype(np.int32)
    slen = np.array([5, 3, 1, 4], np.int32)
    dy_np = r.standard_normal((T, B, U)).astype(np.float32)
    enc = runtime.gnmt_stage(L, U, V, B, S, stash_slots=1); enc.bind(ew)
    att = runtime.gnmt_attention_stage(U, V, B, T, S, stash_slots=1); att.bind(aw)
    dec = runtime.gnmt_decoder_stage(2, U, B, T, stash_slots=1); dec.bind(dw)
    mem = torch.empty(S, B, U, device="cuda"); o1 = torch.empty(T, B, U, device="cuda"); a1 = torch.empty(T, B, U, device="cuda")
    o2 = torch.empty(T, B, U, device="cuda")
    enc.set_lengths(0, dev(slen)); enc.forward(0, dev(src), mem)
    att.set_decoder_inputs(0, dev(tgt), dev(slen), a1); att.forward(0, mem, o1)
    dec.set_attention(0, a1); dec.forward(0, o1, o2)
    d1 = torch.empty_like(o1); dmem = torch.empty_like(mem)
    dec.backward(0, dev(dy_np), d1); att.backward(0, d1, dmem); enc.backward(0, dmem)
    for s in (enc, att, dec):
        s.sync()
    ewt, dwt, awt = og.to_torch(ew, torch.float64, True), og.to_torch(dw, torch.float64, True), oracle_weights(aw)
    m_o = og.encoder_forward(torch.tensor(src), ewt, L, lengths=torch.tensor(slen))
    o1_o, a1_o = og.attention_cell_forward(torch.tensor(tgt), m_o, torch.tensor(slen), awt)
    o2_o = og.decoder_part2_forward(o1_o, a1_o, dwt, 1, 2)
    assert_close(o2, o2_o.detach(), TOL, "chain output")
    params = [(enc, ewt, n) for n in enc.weight_names] + [(att, awt, n) for n in ORDER] + [(dec, dwt, n) for n in dec.weight_names]
    gs = torch.autograd.grad(o2_o, [wt[n] for _, wt, n in params], grad_outputs=torch.tensor(dy_np, dtype=torch.float64))
    for (stg, _, n), g in zip(params, gs):
        assert_close(stg.grads[n], g.reshape(stg.grads[n].shape), TOL, "chain grad " + n)
    for s in (enc, att, dec):
        s.close()
