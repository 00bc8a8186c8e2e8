"""Checkpoint name maps of the reference and a loader that fills a stage's master weights from them.

Mirrors bert/models/bert/modeling_slice.py:82-132 (``get_assigment_map_from_checkpoint``, the reference's
spelling) and xlnet/utils/xlnet_utils.py:107-176 (``get_assignment_map_from_checkpoint``,
``init_from_checkpoint``).  The reference reads TensorFlow checkpoints with ``tf.train``; TensorFlow is not
part of this runtime, so a checkpoint here is any mapping ``variable name -> array`` (``load_checkpoint`` reads
one from ``.npz`` or ``.safetensors`` with loaders that execute nothing from the file).  As with
``tf.train.init_from_checkpoint``, only the variables the assignment map names are overwritten; the others
keep the values the stage was bound with.
"""
import collections
import re

import numpy as np

__all__ = ["get_assigment_map_from_checkpoint", "get_assignment_map_from_checkpoint", "xlnet_stage_assignment",
           "load_checkpoint", "init_from_checkpoint", "init_xlnet_from_checkpoint"]


def _var_name(var):
    name = var if isinstance(var, str) else var.name
    m = re.match("^(.*):\\d+$", name)
    return m.group(1) if m is not None else name


def _ckpt_names(init_vars):
    """Names of a checkpoint given as a mapping, as ``tf.train.list_variables`` pairs ``(name, shape)``, or as names."""
    if hasattr(init_vars, "keys"):
        return list(init_vars.keys())
    return [x if isinstance(x, str) else x[0] for x in init_vars]


def get_assigment_map_from_checkpoint(tvars, init_checkpoint, scope_map=None):
    """Union of the model's variables and the checkpoint's (bert/models/bert/modeling_slice.py:82-132).

    tvars: variable names (``"…:0"`` suffixes are stripped) or objects with ``.name``; init_checkpoint: the
    checkpoint (mapping, ``(name, shape)`` pairs or names).  A checkpoint variable maps to the model variable of
    the same name; with ``scope_map = (old, new)`` it also maps to ``new + name[after the first occurrence of
    old]`` when the model has that variable, and this second match replaces the first, as in the reference.
    Returns ``(assignment_map, initialized_variable_names)``; the latter holds each name and ``name + ":0"``.
    """
    initialized_variable_names = {}
    name_to_variable = collections.OrderedDict()
    for var in tvars:
        name_to_variable[_var_name(var)] = var
    assignment_map = collections.OrderedDict()
    for name in _ckpt_names(init_checkpoint):
        if name in name_to_variable:
            assignment_map[name] = name
            initialized_variable_names[name] = 1
            initialized_variable_names[name + ":0"] = 1
        if scope_map:
            idx = name.find(scope_map[0])
            if idx < 0:
                continue
            new_name = scope_map[1] + name[idx + len(scope_map[0]):]
            if new_name in name_to_variable:
                assignment_map[name] = new_name
                initialized_variable_names[new_name] = 1
                initialized_variable_names[new_name + ":0"] = 1
    return assignment_map, initialized_variable_names


def get_assignment_map_from_checkpoint(tvars, num_layer):
    """Checkpoint name -> Keras variable of the reference's XLNet port (xlnet/utils/xlnet_utils.py:107-166).

    tvars: the Keras-side variables (names or objects with ``.name``); every name the map needs must be there
    (``KeyError`` otherwise, as in the reference).  Layers are 0-based in the checkpoint, 1-based in Keras.
    """
    name_to_variable = collections.OrderedDict()
    for var in tvars:
        name_to_variable[_var_name(var)] = var
    amap = collections.OrderedDict()
    amap["model/transformer/word_embedding/lookup_table"] = name_to_variable["Embed-Token/embeddings"]
    amap["model/transformer/seg_embed"] = name_to_variable["Embed-Segment/seg_emb"]
    amap["model/transformer/r_w_bias"] = name_to_variable["Relative-Bias/bias_context"]
    amap["model/transformer/r_r_bias"] = name_to_variable["Relative-Bias/bias_relative"]
    amap["model/transformer/r_s_bias"] = name_to_variable["Relative-Bias/bias_segment"]
    for i in range(num_layer):
        pre = "model/transformer/layer_%d/" % i
        for p in "qkvro":
            amap[pre + "rel_attn/%s/kernel" % p] = name_to_variable["Attention-%d/%s" % (i + 1, p)]
        amap[pre + "rel_attn/LayerNorm/gamma"] = name_to_variable["Attention-Normal-%d/gamma" % (i + 1)]
        amap[pre + "rel_attn/LayerNorm/beta"] = name_to_variable["Attention-Normal-%d/beta" % (i + 1)]
        for ck, ke in (("layer_1/kernel", "W1"), ("layer_1/bias", "b1"), ("layer_2/kernel", "W2"), ("layer_2/bias", "b2")):
            amap[pre + "ff/" + ck] = name_to_variable["FeedForward-%d/FeedForward-%d_%s" % (i + 1, i + 1, ke)]
        amap[pre + "ff/LayerNorm/gamma"] = name_to_variable["FeedForward-Normal-%d/gamma" % (i + 1)]
        amap[pre + "ff/LayerNorm/beta"] = name_to_variable["FeedForward-Normal-%d/beta" % (i + 1)]
    return amap


# (checkpoint suffix under model/transformer/layer_<l>/, stage suffix under layer_<l>/)
_XL_LAYER = (("rel_attn/q/kernel", "q"), ("rel_attn/k/kernel", "k"), ("rel_attn/v/kernel", "v"), ("rel_attn/r/kernel", "r"),
             ("rel_attn/o/kernel", "o"), ("rel_attn/LayerNorm/gamma", "attn_ln/gamma"), ("rel_attn/LayerNorm/beta", "attn_ln/beta"),
             ("ff/layer_1/kernel", "ff/W1"), ("ff/layer_1/bias", "ff/b1"), ("ff/layer_2/kernel", "ff/W2"),
             ("ff/layer_2/bias", "ff/b2"), ("ff/LayerNorm/gamma", "ff_ln/gamma"), ("ff/LayerNorm/beta", "ff_ln/beta"))
# tables the checkpoint holds once, with a leading [num_layer] axis (xlnet/layers/rel_bias.py:30-55,
# segment_embed.py:23-31); a stage holds one slice per layer
_XL_TABLES = (("model/transformer/r_w_bias", "bias_context"), ("model/transformer/r_r_bias", "bias_relative"),
              ("model/transformer/r_s_bias", "bias_segment"), ("model/transformer/seg_embed", "seg_emb"))


def xlnet_stage_assignment(first_layer, num_layers):
    """Stage weight name -> ``(checkpoint name, layer index or None)`` for an XLNet stage slice holding
    ``num_layers`` layers from ``first_layer`` (same checkpoint names as xlnet/utils/xlnet_utils.py:117-164).
    A layer index means: take slice ``[layer]`` of the checkpoint's ``[num_layer, ...]`` table."""
    out = collections.OrderedDict()
    for l in range(first_layer, first_layer + num_layers):
        for ck, st in _XL_LAYER:
            out["layer_%d/%s" % (l, st)] = ("model/transformer/layer_%d/%s" % (l, ck), None)
        for ck, st in _XL_TABLES:
            out["layer_%d/%s" % (l, st)] = (ck, l)
    return out


def load_checkpoint(path):
    """Reads ``name -> float array`` from ``.npz`` (pickle refused) or ``.safetensors``."""
    if path.endswith(".npz"):
        with np.load(path, allow_pickle=False) as z:
            return collections.OrderedDict((k, z[k]) for k in z.files)
    if path.endswith(".safetensors"):
        from safetensors.numpy import load_file
        return collections.OrderedDict(load_file(path))
    raise ValueError("load_checkpoint: %s is neither .npz nor .safetensors (TensorFlow checkpoints need TensorFlow: "
                     "export them to one of the two first)" % path)


def _assign(stage, name, value):
    import torch
    dst = stage.weights[name]
    src = torch.as_tensor(np.ascontiguousarray(value), dtype=torch.float32)
    if src.numel() != dst.numel():
        raise ValueError("checkpoint tensor for %s has shape %s, stage holds %s" % (name, tuple(src.shape), tuple(dst.shape)))
    dst.copy_(src.reshape(dst.shape))


def init_from_checkpoint(stage, checkpoint, scope_map=None):
    """Overwrites the bound master weights of ``stage`` that the BERT assignment map names and refreshes the
    compute copies.  A tensor may come in the checkpoint's own shape as long as the element count matches.
    Returns ``initialized_variable_names`` (what bert.py logs as ``*INIT_FROM_CKPT*``)."""
    if isinstance(checkpoint, str):
        checkpoint = load_checkpoint(checkpoint)
    if not stage.weights:
        raise RuntimeError("init_from_checkpoint: bind the stage's weights first")
    amap, initialized = get_assigment_map_from_checkpoint(stage.weight_names, checkpoint, scope_map)
    for ck, name in amap.items():
        _assign(stage, name, checkpoint[ck])
    stage.refresh_weights()
    return initialized


def init_xlnet_from_checkpoint(stage, checkpoint, first_layer, num_layers, strict=True):
    """Same for an XLNet stage slice (xlnet/utils/xlnet_utils.py:169-176): per-layer tensors by name, the
    ``[num_layer, ...]`` bias and segment tables sliced at the layer (a table without the layer axis, i.e. one
    shared by all layers, is taken whole).  ``strict`` raises ``KeyError`` on a missing checkpoint variable, as
    the reference's map does; otherwise missing ones are skipped.  Returns the stage names that were set."""
    if isinstance(checkpoint, str):
        checkpoint = load_checkpoint(checkpoint)
    if not stage.weights:
        raise RuntimeError("init_xlnet_from_checkpoint: bind the stage's weights first")
    done = []
    for name, (ck, layer) in xlnet_stage_assignment(first_layer, num_layers).items():
        if name not in stage.weights:
            continue
        if ck not in checkpoint:
            if strict:
                raise KeyError(ck)
            continue
        v = np.asarray(checkpoint[ck])
        if layer is not None and v.size != stage.weights[name].numel():
            if layer >= v.shape[0]:
                raise ValueError("%s has %d layers, the stage needs layer %d" % (ck, v.shape[0], layer))
            v = v[layer]
        _assign(stage, name, v)
        done.append(name)
    stage.refresh_weights()
    return done
