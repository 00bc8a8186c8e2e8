"""Checkpoint name maps (bert/models/bert/modeling_slice.py:82-132, xlnet/utils/xlnet_utils.py:107-176) and the
loader that fills a stage's bound master weights from them.  Host logic only: the stage is a stand-in that holds
CPU tensors under the names the HIP stages report."""
import numpy as np
import pytest
import torch

from dapple_amd import checkpoint as ck
from dapple_amd import synthetic


class FakeStage:
    def __init__(self, weights):
        self.weight_names = list(weights)
        self.weights = {n: torch.as_tensor(np.array(w, dtype=np.float32)) for n, w in weights.items()}
        self.refreshed = 0

    def refresh_weights(self):
        self.refreshed += 1


def test_bert_map_same_names_and_suffix_stripping():
    tvars = ["bert/encoder/layer_0/output/dense/kernel:0", "bert/encoder/layer_0/output/dense/bias", "cls/squad/output_weights:0"]
    init = [("bert/encoder/layer_0/output/dense/kernel", [4, 4]), ("bert/encoder/layer_0/output/dense/bias", [4]),
            ("bert/pooler/dense/kernel", [4, 4]), ("global_step", [])]
    amap, inited = ck.get_assigment_map_from_checkpoint(tvars, init)
    assert list(amap.items()) == [("bert/encoder/layer_0/output/dense/kernel",) * 2, ("bert/encoder/layer_0/output/dense/bias",) * 2]
    assert set(inited) == {"bert/encoder/layer_0/output/dense/kernel", "bert/encoder/layer_0/output/dense/kernel:0",
                           "bert/encoder/layer_0/output/dense/bias", "bert/encoder/layer_0/output/dense/bias:0"}


def test_bert_map_scope_map_replaces_direct_match():
    # a variable that exists under both scopes: the scope-mapped target wins, as the second assignment does in the reference
    tvars = ["bert/a/kernel", "student/a/kernel", "student/b/kernel"]
    init = ["bert/a/kernel", "bert/b/kernel", "bert/c/kernel", "other/a/kernel"]
    amap, inited = ck.get_assigment_map_from_checkpoint(tvars, init, scope_map=("bert/", "student/"))
    assert dict(amap) == {"bert/a/kernel": "student/a/kernel", "bert/b/kernel": "student/b/kernel"}
    assert "bert/a/kernel" in inited and "student/a/kernel:0" in inited and "student/b/kernel" in inited
    assert "bert/c/kernel" not in inited


def test_bert_map_scope_found_inside_name():
    # the reference cuts at the FIRST occurrence of the old scope, wherever it is in the name
    amap, _ = ck.get_assigment_map_from_checkpoint(["new/x"], ["prefix/old/x"], scope_map=("old/", "new/"))
    assert dict(amap) == {"prefix/old/x": "new/x"}


def _keras_names(num_layer):
    names = ["Embed-Token/embeddings:0", "Embed-Segment/seg_emb:0", "Relative-Bias/bias_context:0",
             "Relative-Bias/bias_relative:0", "Relative-Bias/bias_segment:0"]
    for i in range(1, num_layer + 1):
        names += ["Attention-%d/%s:0" % (i, p) for p in "qkvro"]
        names += ["Attention-Normal-%d/gamma:0" % i, "Attention-Normal-%d/beta:0" % i]
        names += ["FeedForward-%d/FeedForward-%d_%s:0" % (i, i, s) for s in ("W1", "b1", "W2", "b2")]
        names += ["FeedForward-Normal-%d/gamma:0" % i, "FeedForward-Normal-%d/beta:0" % i]
    return names


def test_xlnet_keras_map():
    amap = ck.get_assignment_map_from_checkpoint(_keras_names(3), 3)
    assert len(amap) == 5 + 3 * 13
    assert amap["model/transformer/word_embedding/lookup_table"] == "Embed-Token/embeddings:0"
    assert amap["model/transformer/r_s_bias"] == "Relative-Bias/bias_segment:0"
    assert amap["model/transformer/layer_0/rel_attn/q/kernel"] == "Attention-1/q:0"          # 0-based -> 1-based
    assert amap["model/transformer/layer_2/ff/layer_2/bias"] == "FeedForward-3/FeedForward-3_b2:0"
    assert amap["model/transformer/layer_1/rel_attn/LayerNorm/beta"] == "Attention-Normal-2/beta:0"
    with pytest.raises(KeyError):
        ck.get_assignment_map_from_checkpoint(_keras_names(2), 3)


def test_xlnet_stage_assignment_covers_every_stage_weight():
    H, N, F = 64, 4, 128
    names = list(synthetic.xlnet_weights(0, 2, H, N, F, first_layer=3))
    amap = ck.xlnet_stage_assignment(3, 2)
    assert sorted(amap) == sorted(names)
    assert amap["layer_4/bias_context"] == ("model/transformer/r_w_bias", 4)
    assert amap["layer_3/ff/W1"] == ("model/transformer/layer_3/ff/layer_1/kernel", None)
    # the checkpoint side is the key set of the reference's own map
    ref_keys = set(ck.get_assignment_map_from_checkpoint(_keras_names(5), 5))
    assert {c for c, _ in amap.values()} <= ref_keys


def test_init_from_checkpoint_bert(tmp_path):
    w = synthetic.bert_weights(1, 2, 32, 64, stddev=0.05)
    stage = FakeStage({n: np.zeros_like(v) for n, v in w.items()})
    keep = "bert/encoder/layer_1/output/dense/bias"
    ckpt = {n: v for n, v in w.items() if n != keep}
    ckpt["bert/pooler/dense/kernel"] = np.ones((32, 32), np.float32)      # not a stage variable: ignored
    path = str(tmp_path / "bert.npz")
    np.savez(path, **ckpt)
    stage.weights[keep].fill_(7.0)
    inited = ck.init_from_checkpoint(stage, path)
    assert stage.refreshed == 1
    for n, v in w.items():
        if n == keep:
            assert keep not in inited and torch.all(stage.weights[n] == 7.0)   # untouched, as tf.train.init_from_checkpoint leaves it
        else:
            assert n in inited and n + ":0" in inited
            np.testing.assert_array_equal(stage.weights[n].numpy(), v)


def test_init_from_checkpoint_scope_and_shape_errors():
    stage = FakeStage({"bert/encoder/layer_0/output/dense/kernel": np.zeros((4, 6))})
    src = np.arange(24, dtype=np.float32)
    ck.init_from_checkpoint(stage, {"teacher/encoder/layer_0/output/dense/kernel": src.reshape(2, 12)}, scope_map=("teacher/", "bert/"))
    np.testing.assert_array_equal(stage.weights["bert/encoder/layer_0/output/dense/kernel"].numpy().ravel(), src)
    with pytest.raises(ValueError):
        ck.init_from_checkpoint(stage, {"bert/encoder/layer_0/output/dense/kernel": np.zeros((4, 5))})
    empty = FakeStage({})
    with pytest.raises(RuntimeError):
        ck.init_from_checkpoint(empty, {})


def test_init_xlnet_from_checkpoint_slices_layer_tables():
    H, N, F, NL = 64, 4, 128, 6
    D = H // N
    rng = np.random.default_rng(0)
    ckpt = {"model/transformer/r_w_bias": rng.standard_normal((NL, N, D)).astype(np.float32),
            "model/transformer/r_r_bias": rng.standard_normal((NL, N, D)).astype(np.float32),
            "model/transformer/r_s_bias": rng.standard_normal((N, D)).astype(np.float32),     # tied: no layer axis
            "model/transformer/seg_embed": rng.standard_normal((NL, 2, N, D)).astype(np.float32)}
    for l in range(NL):
        pre = "model/transformer/layer_%d/" % l
        for p in "qkvr":
            ckpt[pre + "rel_attn/%s/kernel" % p] = rng.standard_normal((H, N, D)).astype(np.float32)
        ckpt[pre + "rel_attn/o/kernel"] = rng.standard_normal((H, N, D)).astype(np.float32)
        for s, shp in (("rel_attn/LayerNorm/gamma", (H,)), ("rel_attn/LayerNorm/beta", (H,)), ("ff/layer_1/kernel", (H, F)),
                       ("ff/layer_1/bias", (F,)), ("ff/layer_2/kernel", (F, H)), ("ff/layer_2/bias", (H,)),
                       ("ff/LayerNorm/gamma", (H,)), ("ff/LayerNorm/beta", (H,))):
            ckpt[pre + s] = rng.standard_normal(shp).astype(np.float32)
    stage = FakeStage({n: np.zeros_like(v) for n, v in synthetic.xlnet_weights(0, 2, H, N, F, first_layer=3).items()})
    done = ck.init_xlnet_from_checkpoint(stage, ckpt, first_layer=3, num_layers=2)
    assert sorted(done) == sorted(stage.weight_names) and stage.refreshed == 1
    np.testing.assert_array_equal(stage.weights["layer_4/bias_context"].numpy(), ckpt["model/transformer/r_w_bias"][4].reshape(H))
    np.testing.assert_array_equal(stage.weights["layer_3/bias_segment"].numpy(), ckpt["model/transformer/r_s_bias"].reshape(H))
    np.testing.assert_array_equal(stage.weights["layer_3/seg_emb"].numpy(), ckpt["model/transformer/seg_embed"][3].reshape(2, H))
    np.testing.assert_array_equal(stage.weights["layer_4/q"].numpy(), ckpt["model/transformer/layer_4/rel_attn/q/kernel"].reshape(H, H))
    np.testing.assert_array_equal(stage.weights["layer_3/ff/W2"].numpy(), ckpt["model/transformer/layer_3/ff/layer_2/kernel"])
    del ckpt["model/transformer/layer_4/ff/layer_2/bias"]
    with pytest.raises(KeyError):
        ck.init_xlnet_from_checkpoint(stage, ckpt, 3, 2)
    assert "layer_4/ff/b2" not in ck.init_xlnet_from_checkpoint(stage, ckpt, 3, 2, strict=False)
    late = FakeStage({n: np.zeros_like(v) for n, v in synthetic.xlnet_weights(0, 2, H, N, F, first_layer=5).items()})
    with pytest.raises(ValueError):
        ck.init_xlnet_from_checkpoint(late, ckpt, 5, 2, strict=False)       # layer 6 of a 6-layer table


@pytest.mark.gpu
def test_init_from_checkpoint_on_a_bert_stage_gpu():
    """A stage bound with other values and then initialised from a checkpoint gives bit-identical output to a stage
    bound with the checkpoint's values (the compute copies are refreshed by the loader)."""
    from dapple_amd import runtime
    L, H, N, F, B, S = 2, 128, 4, 512, 2, 32
    w = synthetic.bert_weights(1, L, H, F, stddev=0.05, perturb=True)
    other = synthetic.bert_weights(9, L, H, F, stddev=0.05, perturb=True)
    x = torch.as_tensor(synthetic.bert_activation_inputs(2, 1, B, S, H)[0]).cuda().bfloat16()
    outs = []
    for first, load in ((w, False), (other, True)):
        stage = runtime.bert_stage(L, H, N, F, B, S, "bf16", stash_slots=1)
        stage.bind(first)
        if load:
            inited = ck.init_from_checkpoint(stage, dict(w))
            assert all(n in inited for n in stage.weight_names)
        out = torch.empty(B * S, H, dtype=torch.bfloat16, device="cuda")
        stage.forward(0, x, out)
        stage.sync()
        outs.append(out.float().cpu())
        stage.close()
    assert torch.equal(outs[0], outs[1])
