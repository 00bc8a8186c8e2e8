"""Pins the GNMT encoder oracle against torch's LSTM (gate blocks permuted), an explicit loop and
the kernel shape the reference's own test holds."""
import numpy as np
import torch

from dapple_amd import synthetic
from oracle import gnmt as og

D = torch.float64


def _to_torch_lstm(kernel, bias, n_in, forget_bias):
    """TF BasicLSTMCell kernel [in+U,4U] gate order i,j,f,o -> torch weight_ih/hh, bias; torch order i,f,g,o."""
    U = kernel.shape[1] // 4
    i, j, f, o = kernel.chunk(4, 1)
    k = torch.cat([i, f, j, o], 1)
    bi, bj, bf, bo = bias.chunk(4)
    b = torch.cat([bi, bf + forget_bias, bj, bo])
    return k[:n_in].t().contiguous(), k[n_in:].t().contiguous(), b, U


def test_cell_matches_torch_lstmcell_and_kernel_layout():
    I, U, B = 5, 5, 3
    kernel = torch.randn(I + U, 4 * U, dtype=D)
    assert tuple(kernel.shape) == (10, 20)              # gnmt/nmt/model_test.py:86 last_enc_weight shape
    bias = torch.randn(4 * U, dtype=D)
    x, h, c = torch.randn(B, I, dtype=D), torch.randn(B, U, dtype=D), torch.randn(B, U, dtype=D)
    h1, c1 = og.lstm_cell(x, h, c, kernel, bias, forget_bias=1.0)
    wih, whh, b, _ = _to_torch_lstm(kernel, bias, I, 1.0)
    cell = torch.nn.LSTMCell(I, U).double()
    with torch.no_grad():
        cell.weight_ih.copy_(wih); cell.weight_hh.copy_(whh); cell.bias_ih.copy_(b); cell.bias_hh.zero_()
    h2, c2 = cell(x, (h, c))
    assert torch.allclose(h1, h2, atol=1e-12) and torch.allclose(c1, c2, atol=1e-12)
    # forget_bias matters: without it the result differs
    h3, _ = og.lstm_cell(x, h, c, kernel, bias, forget_bias=0.0)
    assert (h3 - h1).abs().max() > 1e-3


def test_bidirectional_layer_matches_torch_lstm():
    T, B, I, U = 6, 2, 4, 4
    x = torch.randn(T, B, I, dtype=D)
    ks = [torch.randn(I + U, 4 * U, dtype=D) * 0.5 for _ in range(2)]
    bs = [torch.randn(4 * U, dtype=D) * 0.5 for _ in range(2)]
    fw = og.dynamic_rnn(x, ks[0], bs[0], 1.0)
    bw = og.dynamic_rnn(x, ks[1], bs[1], 1.0, reverse=True)
    lstm = torch.nn.LSTM(I, U, bidirectional=True).double()
    with torch.no_grad():
        for sfx, k, b in (("", ks[0], bs[0]), ("_reverse", ks[1], bs[1])):
            wih, whh, bb, _ = _to_torch_lstm(k, b, I, 1.0)
            getattr(lstm, "weight_ih_l0" + sfx).copy_(wih)
            getattr(lstm, "weight_hh_l0" + sfx).copy_(whh)
            getattr(lstm, "bias_ih_l0" + sfx).copy_(bb)
            getattr(lstm, "bias_hh_l0" + sfx).zero_()
    ref, _ = lstm(x)
    assert torch.allclose(torch.cat([fw, bw], -1), ref, atol=1e-12)


def test_ragged_sequences_match_torch_packed_lstm():
    """sequence_length: zeros past the end, the backward direction starts at the last valid step
    (torch.nn.LSTM on a packed sequence does exactly that), including a sequence of length 1 and a full one."""
    T, B, I, U = 7, 4, 3, 5
    x = torch.randn(T, B, I, dtype=D)
    lengths = torch.tensor([7, 1, 4, 6])
    ks = [torch.randn(I + U, 4 * U, dtype=D) * 0.5 for _ in range(2)]
    bs = [torch.randn(4 * U, dtype=D) * 0.5 for _ in range(2)]
    fw = og.dynamic_rnn(x, ks[0], bs[0], 1.0, lengths=lengths)
    bw = og.dynamic_rnn(x, ks[1], bs[1], 1.0, reverse=True, lengths=lengths)
    lstm = torch.nn.LSTM(I, U, bidirectional=True).double()
    with torch.no_grad():
        for sfx, k, b in (("", ks[0], bs[0]), ("_reverse", ks[1], bs[1])):
            wih, whh, bb, _ = _to_torch_lstm(k, b, I, 1.0)
            getattr(lstm, "weight_ih_l0" + sfx).copy_(wih)
            getattr(lstm, "weight_hh_l0" + sfx).copy_(whh)
            getattr(lstm, "bias_ih_l0" + sfx).copy_(bb)
            getattr(lstm, "bias_hh_l0" + sfx).zero_()
    packed = torch.nn.utils.rnn.pack_padded_sequence(x, lengths, enforce_sorted=False)
    ref, _ = torch.nn.utils.rnn.pad_packed_sequence(lstm(packed)[0], total_length=T)
    assert torch.allclose(torch.cat([fw, bw], -1), ref, atol=1e-12)
    for b in range(B):
        assert float(fw[lengths[b]:, b].abs().max() if lengths[b] < T else 0.0) == 0.0
    # a residual layer emits zeros past the end too (the wrapped cell's output is what dynamic_rnn replaces)
    k2, b2 = torch.randn(U + U, 4 * U, dtype=D) * 0.5, torch.randn(4 * U, dtype=D) * 0.5
    y = og.dynamic_rnn(fw, k2, b2, 1.0, lengths=lengths, residual=True)
    assert float(y[1:, 1].abs().max()) == 0.0 and float(y[0, 1].abs().max()) > 0.0
    # lengths that cover everything change nothing; zero length gives all zeros
    full = og.dynamic_rnn(x, ks[0], bs[0], 1.0, lengths=torch.full((B,), T))
    assert torch.equal(full, og.dynamic_rnn(x, ks[0], bs[0], 1.0))
    assert float(og.dynamic_rnn(x, ks[0], bs[0], 1.0, lengths=torch.zeros(B, dtype=torch.long)).abs().max()) == 0.0


def test_encoder_structure_residual_from_third_layer():
    T, B, U, V, L = 4, 2, 4, 9, 4
    w = og.to_torch(synthetic.gnmt_weights(1, L, U, V, init_weight=0.5, perturb=True))
    ids = torch.randint(0, V, (B, T), dtype=torch.int32)
    out = og.encoder_forward(ids, w, L)
    assert out.shape == (T, B, U)
    # explicit restatement: bi layer -> uni 1 (input 2U, no residual) -> uni 2, 3 (residual)
    scopes = synthetic.gnmt_cell_scopes(L)
    assert w[scopes[2] + "/kernel"].shape == (3 * U, 4 * U) and w[scopes[3] + "/kernel"].shape == (2 * U, 4 * U)
    emb = w[og.EMB][ids.long().t()]
    x = torch.cat([og.dynamic_rnn(emb, w[scopes[0] + "/kernel"], w[scopes[0] + "/bias"]),
                   og.dynamic_rnn(emb, w[scopes[1] + "/kernel"], w[scopes[1] + "/bias"], reverse=True)], -1)
    x = og.dynamic_rnn(x, w[scopes[2] + "/kernel"], w[scopes[2] + "/bias"])
    for s in scopes[3:]:
        x = og.dynamic_rnn(x, w[s + "/kernel"], w[s + "/bias"]) + x
    assert torch.equal(out, x)
    assert [c[0] for c in og.cell_names(L)] == scopes


def test_parameter_count_of_config():
    # the GNMT-16 encoder configuration = 79.7 M LSTM parameters + 32000 x 1024 embedding
    w = synthetic.gnmt_weights(0, 8, 1024, 32)          # tiny vocab: count the cells only
    cells = sum(v.size for k, v in w.items() if "embedding" not in k)
    assert cells == 2 * (2048 * 4096 + 4096) + (3072 * 4096 + 4096) + 6 * (2048 * 4096 + 4096)
    assert abs(cells - 79.7e6) < 0.1e6


def test_decoder_part2_matches_lstmcell_on_the_concatenated_input():
    torch.manual_seed(7)
    T, B, U = 4, 3, 5
    x = torch.randn(T, B, U, dtype=torch.float64)
    att = torch.randn(T, B, U, dtype=torch.float64, requires_grad=True)
    cells = og.decoder_cell_names(1, 3)
    assert [r for _, r in cells] == [False, True, True] and cells[0][0].endswith("multi_rnn_cell_part2/cell_1/basic_lstm_cell")
    w = {}
    for scope, _ in cells:
        w[scope + "/kernel"] = (torch.randn(3 * U, 4 * U, dtype=torch.float64) * 0.3).requires_grad_(True)
        w[scope + "/bias"] = torch.randn(4 * U, dtype=torch.float64) * 0.1
    out = og.decoder_part2_forward(x, att, w, 1, 3, forget_bias=1.0)
    # library cells: torch gate order i, f, g, o; TF order i, j(=g), f, o; forget_bias folded into the bias
    perm = torch.cat([torch.arange(0, U), torch.arange(2 * U, 3 * U), torch.arange(U, 2 * U), torch.arange(3 * U, 4 * U)])
    lib = []
    for scope, _ in cells:
        c = torch.nn.LSTMCell(2 * U, U).double()
        k, b = w[scope + "/kernel"].detach(), w[scope + "/bias"].clone()
        b[2 * U:3 * U] += 1.0
        with torch.no_grad():
            c.weight_ih.copy_(k[:2 * U, perm].t()); c.weight_hh.copy_(k[2 * U:, perm].t())
            c.bias_ih.copy_(b[perm]); c.bias_hh.zero_()
        lib.append(c)
    st = [(torch.zeros(B, U, dtype=torch.float64), torch.zeros(B, U, dtype=torch.float64)) for _ in cells]
    for t in range(T):
        cur = x[t]
        for i, (_, residual) in enumerate(cells):
            h, c = lib[i](torch.cat([cur, att[t].detach()], -1), st[i])
            st[i] = (h, c)
            cur = h + cur if residual else h
        assert torch.allclose(out[t], cur, atol=1e-12)
    # the attention is a constant of the graph; the kernel rows that multiply it do get a gradient
    gk = torch.autograd.grad(out.sum(), [w[cells[0][0] + "/kernel"]], retain_graph=True)[0]
    assert float(gk[U:2 * U].abs().max()) > 0
    assert torch.autograd.grad(out.sum(), [att], allow_unused=True)[0] is None
    # zeros for the attention (the variable's initial value) = dropping those kernel rows
    out0 = og.decoder_part2_forward(x, None, w, 1, 3)
    w1 = {k: (torch.cat([v[:U], torch.zeros(U, 4 * U, dtype=torch.float64), v[2 * U:]]) if k.endswith("kernel") else v) for k, v in w.items()}
    assert torch.allclose(out0, og.decoder_part2_forward(x, att, w1, 1, 3), atol=1e-12)


def test_nmt_loss_matches_library_cross_entropy():
    torch.manual_seed(8)
    T, B, U, V = 5, 3, 4, 7
    outs = torch.randn(T, B, U, dtype=torch.float64)
    k = torch.randn(U, V, dtype=torch.float64)
    tgt = torch.randint(0, V, (B, T))
    lens = torch.tensor([5, 2, 0])
    loss, logits = og.nmt_loss(outs, k, tgt, lens)
    tot = 0.0
    for b in range(B):
        n = int(lens[b])
        if n:
            tot += torch.nn.functional.cross_entropy(logits[:n, b], tgt[b, :n], reduction="sum").item()
    assert abs(loss.item() - tot / B) < 1e-12
    assert torch.allclose(logits[2, 1], outs[2, 1] @ k)


def _attention_case(seed, T, B, S, U, V):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.rand(*s, generator=g, dtype=torch.float64) * 2 - 1
    w = {og.EMB_DEC: r(V, U) * 0.5, og.ATT_CELL + "/kernel": r(3 * U, 4 * U) * 0.4, og.ATT_CELL + "/bias": r(4 * U) * 0.1,
         og.ATT_MEM: r(U, U) * 0.5, og.ATT_Q: r(U, U) * 0.5, og.ATT_V: r(U), og.ATT_G: torch.tensor((1.0 / U) ** 0.5, dtype=torch.float64),
         og.ATT_B: r(U) * 0.1}
    ids = torch.randint(0, V, (B, T), generator=g)
    mem = r(S, B, U)
    return w, ids, mem


def test_attention_cell_against_library_pieces_and_scalar_loops():
    import math
    T, B, S, U, V = 3, 2, 4, 3, 6
    w, ids, mem = _attention_case(9, T, B, S, U, V)
    lens = torch.tensor([4, 2])
    outs, atts = og.attention_cell_forward(ids, mem, lens, w)
    perm = torch.cat([torch.arange(0, U), torch.arange(2 * U, 3 * U), torch.arange(U, 2 * U), torch.arange(3 * U, 4 * U)])
    cell = torch.nn.LSTMCell(2 * U, U).double()
    k, b = w[og.ATT_CELL + "/kernel"], w[og.ATT_CELL + "/bias"].clone()
    b[2 * U:3 * U] += 1.0
    with torch.no_grad():
        cell.weight_ih.copy_(k[:2 * U, perm].t()); cell.weight_hh.copy_(k[2 * U:, perm].t()); cell.bias_ih.copy_(b[perm]); cell.bias_hh.zero_()
    h = c = torch.zeros(B, U, dtype=torch.float64)
    att = torch.zeros(B, U, dtype=torch.float64)
    v = w[og.ATT_V].tolist()
    vn = math.sqrt(sum(x * x for x in v))
    for t in range(T):
        h, c = cell(torch.cat([w[og.EMB_DEC][ids[:, t]], att], -1), (h, c))
        assert torch.allclose(outs[t], h, atol=1e-12)
        new_att = torch.zeros(B, U, dtype=torch.float64)
        for bb in range(B):
            pq = [sum(h[bb, i].item() * w[og.ATT_Q][i, u].item() for i in range(U)) for u in range(U)]
            sc = []
            for j in range(int(lens[bb])):
                key = [sum(mem[j, bb, i].item() * w[og.ATT_MEM][i, u].item() for i in range(U)) for u in range(U)]
                sc.append(sum(w[og.ATT_G].item() * v[u] / vn * math.tanh(key[u] + pq[u] + w[og.ATT_B][u].item()) for u in range(U)))
            mx = max(sc)
            z = sum(math.exp(s - mx) for s in sc)
            for j, s in enumerate(sc):
                new_att[bb] += math.exp(s - mx) / z * mem[j, bb]
        assert torch.allclose(atts[t], new_att, atol=1e-12)
        att = new_att
    # memory past the source length influences nothing
    mem2 = mem.clone(); mem2[2:, 1] += 5.0
    outs2, atts2 = og.attention_cell_forward(ids, mem2, lens, w)
    assert torch.equal(outs, outs2) and torch.equal(atts, atts2)
