"""The mirrored reference interfaces drive the HIP stages (GPU)."""
import types

import numpy as np
import pytest
import torch

from dapple_amd import slices, synthetic
from oracle import bert as ob
from util import assert_close

pytestmark = pytest.mark.gpu


def test_bert_model_slice_stages_like_modeling_test():
    # bert/models/bert/modeling_test.py:114-124 pins the shapes: embedding / sequence output [B, S, H]
    B, S = 2, 8
    cfg = slices.BertConfig(vocab_size=99, hidden_size=32, num_hidden_layers=2, num_attention_heads=4, intermediate_size=64,
                            type_vocab_size=16, max_position_embeddings=64)
    ids = torch.randint(0, 99, (B, S), dtype=torch.int32, device="cuda")
    model = slices.BertModelSlice(cfg, False, ids)
    assert len(model.stages) == cfg.num_hidden_layers + 3
    x = ids
    for f in model.stages[:-1]:
        x = f(x)
    assert model.get_embedding_output().shape == (B, S, 32) and model.get_sequence_output().shape == (B, S, 32)
    assert len(model.get_all_encoder_layers()) == 2
    w = ob.to_torch(model.weights)
    want = ob.stage_forward(ids.cpu(), w, [0, 1], B, S, 4)
    assert_close(x, want, 1e-4, "stages chained")
    # the last entry is pooler_stage (modeling_slice.py:849-868): tanh dense on the first token
    pooled = model.stages[-1](x)
    assert pooled is model.get_pooled_output() and pooled.shape == (B, 32)
    pk, pb = model._pooler_params(x.device)
    first = want.reshape(B, S, 32)[:, 0, :].double()
    assert_close(pooled, torch.tanh(first @ pk.cpu().double() + pb.cpu().double()), 1e-4, "pooler_stage")
    # calling the stages again works: a forward-only call gives its stash slot back without a backward pass
    x2 = ids
    for f in model.stages[:-1]:
        x2 = f(x2)
    assert torch.equal(x2, x)
    bad = slices.BertConfig(vocab_size=9, hidden_size=30, num_attention_heads=4)
    with pytest.raises(ValueError, match="not a multiple of the number of attention"):
        slices.BertModelSlice(bad, False, ids)
    with pytest.raises(ValueError, match="cannot be greater than `max_position_embeddings`"):
        slices.BertModelSlice(slices.BertConfig(vocab_size=9, hidden_size=32, num_attention_heads=4, max_position_embeddings=4), False, ids)


def test_bert_finetune_slice_puts_the_planner_split_on_each_device():
    cfg = slices.BertConfig(vocab_size=50, hidden_size=32, num_hidden_layers=24, num_attention_heads=4, intermediate_size=64,
                            type_vocab_size=2, max_position_embeddings=16)
    ids = torch.randint(0, 50, (2, 8), dtype=torch.int32, device="cuda")
    s0 = slices.BertFinetuneSlice(cfg, 8, False, ids, None, None, None, False, model_type="mrc",
                                  slice_devices="/gpu:0,/gpu:1", local_device=0, dtype="fp32")
    s1 = slices.BertFinetuneSlice(cfg, 8, False, ids, None, None, None, False, model_type="mrc",
                                  slice_devices=["/gpu:0", "/gpu:1"], local_device=1, dtype="fp32")
    assert s0.layers == list(range(11)) and s1.layers == list(range(11, 24))
    # .stages is the model's list of per-op callables (bert.py:414), 27 entries for BERT-24, placed by calc_device
    assert len(s1.stages) == 27 and s1.stages is s1.model.stages
    assert [s1.device_of[i] for i in (0, 12, 13, 26)] == [0, 0, 1, 1]
    assert s0.stage.takes_input_grad is False and s1.stage.takes_input_grad is True
    assert s0.stage.stash_slots == 2 and s1.stage.stash_slots == 1          # K = S - i
    assert s0.stage.weight_names[0] == "bert/embeddings/word_embeddings"
    assert s1.stage.weight_names[0] == "bert/encoder/layer_11/attention/self/query/kernel"
    with pytest.raises(ValueError, match="Cannot use sequence length"):
        slices.BertFinetuneSlice(cfg, 32, False, ids, None, None, None, False)
    # the last device holds the SQuAD output layer (bert.py:467-470): loss from kwargs' positions, and the gradient
    # that feeds the stage's backward pass
    s1.kwargs = {"start_positions": [1, 2], "end_positions": [3, 7]}
    h = torch.randn(2 * 8, 32, device="cuda")
    y = torch.empty_like(h)
    s1.stage.forward(0, h, y)
    dy = s1.build_output_layer_squad(y.reshape(2, 8, 32))
    assert s1.stage_outputs[-1] is s1.loss and 0.0 < float(s1.loss) < 10.0
    assert dy.shape == y.shape and float(s1.d_output_weights.abs().max()) > 0
    s1.stage.backward(0, dy, torch.empty_like(h))
    with pytest.raises(ValueError, match="does not hold"):
        s0.build_output_layer_squad(y)
    # model_type='classification' (bert.py:463-464): pooler + FC over two classes on the last device
    s2 = slices.BertFinetuneSlice(cfg, 8, False, ids, None, None, [1, 0], False, model_type="classification",
                                  slice_devices="/gpu:0,/gpu:1", local_device=1, dtype="fp32")
    s2.stage.forward(0, h, y)
    dy = s2.build_output_layer_classification(y.reshape(2, 8, 32))
    assert s2.stage_outputs[-1] is s2.loss and 0.0 < float(s2.loss) < 10.0
    assert tuple(s2.logits.shape) == (2, 2) and tuple(s2.pooled_output.shape) == (2, 32) and tuple(s2.predictions.shape) == (2,)
    assert float(dy.reshape(2, 8, 32)[:, 1:].abs().max()) == 0.0 and float(dy.reshape(2, 8, 32)[:, 0].abs().max()) > 0
    assert all(float(g.abs().max()) > 0 for g in s2.head_grads)
    s2.stage.backward(0, dy, torch.empty_like(h))
    with pytest.raises(ValueError, match="does not hold"):
        s1.build_output_layer_classification(y)
    # model_type='regression' (bert.py:465-466): pooler + one output, the graph's pairwise squared-error mean
    s3 = slices.BertFinetuneSlice(cfg, 8, False, ids, None, None, [0.5, -1.25], False, model_type="regression",
                                  slice_devices="/gpu:0,/gpu:1", local_device=1, dtype="fp32")
    s3.stage.forward(0, h, y)
    dy = s3.build_output_layer_regression(y.reshape(2, 8, 32))
    assert s3.stage_outputs[-1] is s3.loss and float(s3.loss) > 0.0
    assert tuple(s3.logits.shape) == (2, 1) and tuple(s3.fc_weights.shape) == (32, 1) and s3.predictions is s3.logits
    z, t = s3.logits[:, 0].double().cpu(), torch.tensor([0.5, -1.25], dtype=torch.float64)
    want = ((z[:, None] - t[None, :]) ** 2).mean() + 1e-3 * 0.5 * float((s3.fc_weights.double() ** 2).sum())
    assert abs(float(s3.loss) - float(want)) < 1e-5 * max(1.0, float(want))
    assert float(dy.reshape(2, 8, 32)[:, 1:].abs().max()) == 0.0 and float(dy.reshape(2, 8, 32)[:, 0].abs().max()) > 0
    s3.stage.backward(0, dy, torch.empty_like(h))
    with pytest.raises(ValueError, match="does not hold"):
        s2.build_output_layer_regression(y)
    s0.stage.close(); s1.stage.close(); s3.stage.close()


def test_vgg_xlnet_gnmt_slices_build():
    v = slices.SliceVGG19(num_replica=2)
    assert [n for n, _ in v.layers][-1] == "block3_pool"
    _, outs = v.build(torch.randn(2, 32, 32, 3, device="cuda"), None)
    assert outs[0].shape == (2, 4, 4, 256)
    x = slices.XlnetSlice(32000, 24, 4, 64, 16, 128, 16, False, memory_len=0, local_device=0, batch_size=2, dtype="fp32")
    assert x.layers == list(range(11))
    _, outs = x.build(torch.randn(1, 16, 2, 64, device="cuda"))
    assert outs[0].shape == (1, 16, 2, 64) and torch.isfinite(outs[0]).all()
    assert not x.is_last
    with pytest.raises(ValueError):
        x.xlnet_loss([0, 0], [1, 2], [3, 4], [0.0, 1.0], torch.zeros(2, 16), outs[0][0])
    x.stage.close()
    # the last device: layers 11..23, then XLnetLoss on the content stream; its input gradient feeds the backward pass
    x1 = slices.XlnetSlice(32000, 24, 4, 64, 16, 128, 16, False, memory_len=0, local_device=1, batch_size=2, dtype="fp32", stash_slots=1)
    assert x1.layers == list(range(11, 24)) and x1.is_last
    xin = torch.randn(1, 16, 2, 64, device="cuda")
    y = torch.empty_like(xin)
    x1.stage.forward(0, xin, y)
    dy = x1.xlnet_loss([0, 15], [1, 2], [3, 4], [0.0, 1.0], torch.zeros(2, 16), y[0])
    assert x1.loss.shape == (1,) and torch.isfinite(x1.loss).all() and x1.start_logits.shape == (2, 16) and x1.cls_logits.shape == (2,)
    dxin = torch.empty_like(xin)
    x1.stage.backward(0, dy.reshape(1, 16, 2, 64), dxin)
    x1.stage.sync()
    assert torch.isfinite(dxin).all() and float(dxin.abs().max()) > 0 and float(x1.loss_grads["end_w0"].abs().max()) > 0
    x1.stage.close()
    hp = types.SimpleNamespace(unit_type="lstm", num_units=16, forget_bias=1.0, dropout=0.0, num_encoder_layers=3, src_vocab_size=40)
    g = slices.GNMTEncoderSlice(hp, batch_size=4, src_max_len=5)
    assert [c.residual_connection for c in g.cells] == [False, False, False, True]
    out = g.build_graph(torch.randint(0, 40, (4, 5), device="cuda"))
    assert out.shape == (5, 4, 16)
