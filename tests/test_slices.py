"""Host logic of the mirrored stage-slice interfaces (no GPU): planner splits, config parsing, KATs."""
import json
import types

import pytest

from dapple_amd import runtime, slices


def test_bert_calc_device_matches_reference_splits():
    # bert/models/bert/bert.py:419-430: BERT-24 = 27 stages, 11:13 layers; BERT-48 = 51 stages, 23:25 layers
    d24 = [slices.bert_calc_device(i, 27) for i in range(27)]
    assert d24.count(0) == 13 and d24.count(1) == 14 and d24 == sorted(d24)
    assert sum(1 for i in range(2, 26) if d24[i] == 0) == 11
    d48 = [slices.bert_calc_device(i, 51) for i in range(51)]
    assert sum(1 for i in range(2, 50) if d48[i] == 0) == 23 and sum(1 for i in range(2, 50) if d48[i] == 1) == 25
    with pytest.raises(SystemExit):
        slices.bert_calc_device(0, 15)


def test_xlnet_calc_device_matches_reference_splits():
    # xlnet/models/slice_xlnet.py:106-121: layer l is stage function l + 2; XLNet-36 -> 17 : 19, XLNet-24 -> 11 : 13
    for L, first in ((36, 17), (24, 11)):
        dev = [slices.xlnet_calc_device(l + 2, L) for l in range(L)]
        assert dev.count(0) == first and dev.count(1) == L - first and dev == sorted(dev)


def test_calc_reduction_layers_kat():
    # amoeba_net/network_utils_test.py:28-35
    r = slices.calc_reduction_layers(18, 2)
    assert len(r) == 2 and r[0] == 6 and r[1] == 12


def test_bert_config_round_trip(tmp_path):
    cfg = {"vocab_size": 30522, "hidden_size": 1024, "num_hidden_layers": 48, "num_attention_heads": 16,
           "intermediate_size": 4096, "type_vocab_size": 2, "max_position_embeddings": 512, "hidden_act": "gelu",
           "hidden_dropout_prob": 0.1, "attention_probs_dropout_prob": 0.1, "initializer_range": 0.02}
    p = tmp_path / "bert_config.json"
    p.write_text(json.dumps(cfg))
    c = slices.BertConfig.from_json_file(str(p))
    assert c.to_dict() == cfg and json.loads(c.to_json_string()) == cfg
    assert slices.BertConfig(vocab_size=7).hidden_size == 768          # defaults of modeling_slice.py:649-660


def test_single_cell_dapple_contract():
    hp = types.SimpleNamespace(unit_type="lstm", num_units=8, forget_bias=1.0, dropout=0.0)
    c = slices._single_cell_dapple(hp, "train", 3, residual_connection=True, device_str="/gpu:0")
    assert (c.layer_id, c.num_units, c.forget_bias, c.residual_connection, c.device_str) == (3, 8, 1.0, True, "/gpu:0")
    hp.unit_type = "gru"
    with pytest.raises(ValueError, match="Unknown unit type gru!"):
        slices._single_cell_dapple(hp, "train", 0)


def test_amoeba_shell_and_vgg_replica_check():
    cell = slices.BaseCell(64, ["none"], [1], [0], 1.0, 6, 0, dep_outputs=None)
    assert cell.cut_outputs == []
    with pytest.raises(NotImplementedError):
        slices.build_network(None, 10)
    with pytest.raises(SystemExit):
        slices.SliceVGG19(num_replica=3)


def test_schedule_ops_rules():
    # bert/graph.py:129 (K = S - i) and vgg19/tf-keras-dapple.py:292 (K = 2S - 1 - i)
    assert runtime.schedule_ops(0, 2, 4) == [("F", 0), ("F", 1), ("B", 0), ("F", 2), ("B", 1), ("F", 3), ("B", 2), ("B", 3)]
    assert runtime.schedule_ops(1, 2, 3) == [("F", 0), ("B", 0), ("F", 1), ("B", 1), ("F", 2), ("B", 2)]
    assert [op for op, _ in runtime.schedule_ops(0, 2, 4, "2S-1")][:4] == ["F", "F", "F", "B"]
    assert runtime.stash_depth(0, 2, "2S-1") == 3
    with pytest.raises(ValueError):
        runtime.schedule_ops(2, 2, 4)
    # the product's schedule equals the oracle's closed form and its graph simulation
    from oracle import schedule as osched
    for S, M in ((2, 8), (3, 5), (4, 4)):
        sim = osched.simulate(S, M)
        for i in range(S):
            assert runtime.schedule_ops(i, S, M) == osched.closed_form(i, S, M) == sim[i]
