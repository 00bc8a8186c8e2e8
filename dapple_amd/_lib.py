"""ctypes binding of libdapple_hip.so (the C ABI declared in include/dapple_stage.h).

There is no CPU fallback: if the library is missing or a call fails, this module
raises.  Build it with ``python -m dapple_amd.build`` (hipcc, gfx950).
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libdapple_hip.so")

DS_F32, DS_BF16 = 0, 1
DS_K_MAJOR, DS_MN_MAJOR = 0, 1
DS_EPI_BIAS, DS_EPI_RESIDUAL, DS_EPI_GELU, DS_EPI_DGELU = 1, 2, 4, 8
DS_EPI_OUT_F32, DS_EPI_ACCUM, DS_EPI_RELU, DS_EPI_MASK, DS_EPI_TANH_FORM = 16, 32, 64, 128, 256
DS_EPI_GELU_GRAD, DS_EPI_MUL, DS_EPI_RESIDUAL_F32 = 512, 1024, 2048
DS_VGG_LOSS_AS_WRITTEN, DS_VGG_LOSS_SPARSE_CE = 0, 1
DS_STAGE_BERT, DS_STAGE_VGG19, DS_STAGE_GNMT, DS_STAGE_XLNET = 0, 1, 2, 3


class DappleError(RuntimeError):
    pass


class GemmDesc(C.Structure):
    _fields_ = [
        ("dtype", C.c_int), ("a_major", C.c_int), ("b_major", C.c_int),
        ("m", C.c_int), ("n", C.c_int), ("k", C.c_int),
        ("lda", C.c_int64), ("ldb", C.c_int64), ("ldc", C.c_int64),
        ("batch", C.c_int), ("batch_inner", C.c_int),
        ("a_stride_outer", C.c_int64), ("a_stride_inner", C.c_int64),
        ("b_stride_outer", C.c_int64), ("b_stride_inner", C.c_int64),
        ("c_stride_outer", C.c_int64), ("c_stride_inner", C.c_int64),
        ("flags", C.c_int), ("alpha", C.c_float),
        ("a", C.c_void_p), ("b", C.c_void_p), ("c", C.c_void_p),
        ("bias", C.c_void_p), ("residual", C.c_void_p), ("c2", C.c_void_p),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
        ("k_segment", C.c_int), ("a_segment_stride", C.c_int64), ("b_segment_stride", C.c_int64),
    ]


class StageCfg(C.Structure):
    _fields_ = [
        ("kind", C.c_int), ("dtype", C.c_int), ("num_layers", C.c_int),
        ("hidden", C.c_int), ("heads", C.c_int), ("ffn", C.c_int),
        ("batch", C.c_int), ("seq", C.c_int), ("with_embedding", C.c_int),
        ("vocab", C.c_int), ("type_vocab", C.c_int), ("max_pos", C.c_int),
        ("ln_eps", C.c_float), ("stash_slots", C.c_int), ("first_layer", C.c_int),
        ("wgrad_group", C.c_int), ("residual_fp32", C.c_int), ("reserved", C.c_int * 5),
    ]


class VggCfg(C.Structure):
    _fields_ = [
        ("dtype", C.c_int), ("batch", C.c_int), ("height", C.c_int), ("width", C.c_int), ("in_channels", C.c_int),
        ("num_ops", C.c_int), ("ops", C.c_int * 40), ("stash_slots", C.c_int), ("need_input_grad", C.c_int),
        ("reserved", C.c_int * 8),
    ]


class GnmtCfg(C.Structure):
    _fields_ = [
        ("dtype", C.c_int), ("num_layers", C.c_int), ("units", C.c_int), ("vocab", C.c_int), ("batch", C.c_int),
        ("seq", C.c_int), ("forget_bias", C.c_float), ("stash_slots", C.c_int), ("part", C.c_int), ("first_layer", C.c_int),
        ("src_seq", C.c_int), ("reserved", C.c_int * 5),
    ]


XLNET_HEAD_TENSORS = ("start_w", "start_b", "end_w0", "end_b0", "ln_gamma", "ln_beta", "end_w1", "end_b1", "ans_w0", "ans_b0",
                      "ans_w1")


class XlnetHeadParams(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in XLNET_HEAD_TENSORS]


class XlnetCfg(C.Structure):
    _fields_ = [
        ("dtype", C.c_int), ("num_layers", C.c_int), ("hidden", C.c_int), ("heads", C.c_int), ("ffn", C.c_int),
        ("batch", C.c_int), ("seq", C.c_int), ("mem_len", C.c_int), ("streams", C.c_int), ("ln_eps", C.c_float),
        ("first_layer", C.c_int), ("stash_slots", C.c_int), ("fused_attention", C.c_int), ("residual_fp32", C.c_int),
        ("wgrad_group", C.c_int), ("reserved", C.c_int * 5),
    ]


# name -> (restype, argtypes); every symbol include/dapple_stage.h declares
PROTOTYPES = {
    "ds_last_error": (C.c_char_p, []),
    "ds_build_target": (C.c_char_p, []),
    "ds_profile_enable": (C.c_int, [C.c_int]),
    "ds_profile_dump": (C.c_int, [C.c_char_p, C.c_size_t]),
    "ds_grad_accumulate": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]),
    "ds_cast_f32_to_bf16": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "ds_cast_bf16_to_f32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "ds_gemm": (C.c_int, [C.POINTER(GemmDesc), C.c_void_p]),
    "ds_gemm_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int]),
    "ds_gemm_grouped": (C.c_int, [C.POINTER(GemmDesc), C.POINTER(C.c_int), C.c_int, C.c_void_p]),
    "ds_vgg_stage_read_activation": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_size_t]),
    "ds_layernorm_fwd_mixed": (C.c_int, [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_void_p,
                                          C.c_void_p, C.c_void_p]),
    "ds_layernorm_bwd_mixed": (C.c_int, [C.c_int, C.c_int] + [C.c_void_p] * 11),
    "ds_layernorm_param_grads_mixed": (C.c_int, [C.c_int, C.c_int] + [C.c_void_p] * 8),
    "ds_layernorm_bwd_mixed_rows": (C.c_int, [C.c_int, C.c_int] + [C.c_void_p] * 9),
    "ds_layernorm_param_grads_exact": (C.c_int, [C.c_int, C.c_int] + [C.c_void_p] * 9),
    "ds_gemm_static_scratch": (C.c_int, [C.POINTER(GemmDesc), C.c_void_p]),
    "ds_gemm_static_scratch_init": (C.c_int, []),
    "ds_vgg_head_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int]),
    "ds_vgg_head": (C.c_int, [C.c_int] * 4 + [C.c_void_p] * 8 + [C.c_int, C.c_float] + [C.c_void_p] * 10 + [C.c_size_t, C.c_void_p]),
    "ds_pooler": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_stage_release_slot": (C.c_int, [C.c_void_p, C.c_int]),
    "ds_relu_fwd": (C.c_int, [C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_relu_bwd": (C.c_int, [C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
    "ds_add": (C.c_int, [C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_copy2d": (C.c_int, [C.c_int64, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_int, C.c_void_p]),
    "ds_batchnorm_workspace_bytes": (C.c_size_t, [C.c_int]),
    "ds_batchnorm_train_fwd": (C.c_int, [C.c_int64, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_float] + [C.c_void_p] * 5 +
                               [C.c_float, C.c_void_p, C.c_void_p]),
    "ds_batchnorm_train_bwd": (C.c_int, [C.c_int64, C.c_int] + [C.c_void_p] * 6 + [C.c_int] + [C.c_void_p] * 4),
    "ds_pool3x3_fwd": (C.c_int, [C.c_int] * 5 + [C.c_void_p] * 3),
    "ds_pool3x3_bwd": (C.c_int, [C.c_int] * 5 + [C.c_void_p] * 3 + [C.c_int, C.c_void_p]),
    "ds_depthwise_conv_fwd": (C.c_int, [C.c_int] * 5 + [C.c_void_p] * 4),
    "ds_depthwise_conv_bwd": (C.c_int, [C.c_int] * 5 + [C.c_void_p] * 4 + [C.c_int, C.c_void_p, C.c_void_p]),
    "ds_gather1d": (C.c_int, [C.c_int] * 6 + [C.c_void_p] * 3),
    "ds_scatter1d": (C.c_int, [C.c_int] * 6 + [C.c_void_p] * 2 + [C.c_int, C.c_void_p]),
    "ds_lstm_cell_fwd": (C.c_int, [C.c_int, C.c_int, C.c_float] + [C.c_void_p] * 7),
    "ds_lstm_cell_bwd": (C.c_int, [C.c_int, C.c_int] + [C.c_void_p] * 5 + [C.c_int, C.c_void_p, C.c_void_p]),
    "ds_layernorm_fwd": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_float,
                                   C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_layernorm_bwd": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                   C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_layernorm_param_grads": (C.c_int, [C.c_int, C.c_int, C.c_int] + [C.c_void_p] * 8),
    "ds_softmax_fwd": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_float, C.c_void_p,
                                 C.c_float, C.c_void_p, C.c_void_p]),
    "ds_softmax_bwd": (C.c_int, [C.c_int, C.c_int64, C.c_int, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p,
                                 C.c_void_p]),
    "ds_attention_fwd": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_float,
                                   C.c_float, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_attention_bwd": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_float,
                                   C.c_float, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_attention_key_mean": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]),
    "ds_attention_bwd_centered": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_float,
                                            C.c_float, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_colsum_accum": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]),
    "ds_xlnet_scores_meta_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int]),
    "ds_xlnet_scores_pack": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_xlnet_bias_q": (C.c_int, [C.c_int, C.c_int, C.c_int] + [C.c_void_p] * 10),
    "ds_xlnet_scores_fwd": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_void_p]),
    "ds_xlnet_scores_bwd": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_void_p, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_conv3x3_fwd": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                 C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_conv3x3_wgrad": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                   C.c_void_p, C.c_void_p]),
    "ds_conv3x3_flip": (C.c_int, [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_maxpool2x2_fwd": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_maxpool2x2_bwd": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                    C.c_void_p]),
    "ds_vgg_stage_create": (C.c_int, [C.POINTER(VggCfg), C.c_void_p, C.POINTER(C.c_void_p)]),
    "ds_gnmt_stage_create": (C.c_int, [C.POINTER(GnmtCfg), C.c_void_p, C.POINTER(C.c_void_p)]),
    "ds_gnmt_stage_set_lengths": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
    "ds_gnmt_stage_set_attention": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
    "ds_gnmt_stage_set_decoder_inputs": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_xlnet_stage_create": (C.c_int, [C.POINTER(XlnetCfg), C.c_void_p, C.POINTER(C.c_void_p)]),
    "ds_xlnet_stage_set_inputs": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_stage_create": (C.c_int, [C.POINTER(StageCfg), C.c_void_p, C.POINTER(C.c_void_p)]),
    "ds_stage_destroy": (C.c_int, [C.c_void_p]),
    "ds_stage_num_weights": (C.c_int, [C.c_void_p]),
    "ds_stage_weight_info": (C.c_int, [C.c_void_p, C.c_int, C.c_char_p, C.c_size_t, C.POINTER(C.c_int64),
                                       C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "ds_stage_bind_weights": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p)]),
    "ds_stage_refresh_weights": (C.c_int, [C.c_void_p]),
    "ds_stage_forward": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_stage_set_token_types": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
    "ds_stage_backward": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "ds_stage_forward_backward": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "ds_stage_backward_after": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_stage_backward_event": (C.c_void_p, [C.c_void_p, C.c_int]),
    "ds_stage_wait_backward": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
    "ds_stage_workspace_bytes": (C.c_size_t, [C.c_void_p]),
    "ds_stage_stash_bytes": (C.c_size_t, [C.c_void_p, C.c_int]),
    "ds_stage_sync": (C.c_int, [C.c_void_p]),
    "ds_stage_overlap_supported": (C.c_int, [C.c_void_p]),
    "ds_stage_enable_overlap": (C.c_int, [C.c_void_p, C.c_int]),
    "ds_stage_join": (C.c_int, [C.c_void_p]),
    "ds_squad_head": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                C.c_float, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ds_classifier_head": (C.c_int, [C.c_int] * 5 + [C.c_void_p] * 6 + [C.c_float, C.c_float] + [C.c_void_p] * 11),
    "ds_regression_head": (C.c_int, [C.c_int] * 4 + [C.c_void_p] * 6 + [C.c_float, C.c_float] + [C.c_void_p] * 11),
    "ds_nmt_loss_head_workspace_bytes": (C.c_size_t, [C.c_int] * 3),
    "ds_nmt_loss_head": (C.c_int, [C.c_int] * 4 + [C.c_void_p] * 4 + [C.c_int, C.c_float] + [C.c_void_p] * 4 + [C.c_size_t, C.c_void_p]),
    "ds_xlnet_squad_head_workspace_bytes": (C.c_size_t, [C.c_int] * 4),
    "ds_xlnet_squad_head": (C.c_int, [C.c_int] * 4 + [C.c_void_p, C.POINTER(XlnetHeadParams)] + [C.c_void_p] * 6 + [C.c_float] +
                            [C.c_void_p] * 5 + [C.POINTER(XlnetHeadParams), C.c_void_p, C.c_size_t, C.c_void_p]),
    "ds_grad_sqnorm_accum": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p]),
    "ds_optim_plan_create": (C.c_int, [C.c_int, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_float),
                                        C.POINTER(C.c_void_p)]),
    "ds_optim_plan_destroy": (C.c_int, [C.c_void_p]),
    "ds_adam_step": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double, C.c_double, C.c_double,
                               C.c_double, C.c_void_p, C.c_float, C.c_void_p]),
    "ds_sgd_step": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_double, C.c_void_p, C.c_float, C.c_void_p]),
}

_lib = None


def load():
    """Loads the shared library and sets the prototypes; raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise DappleError("%s not found: build it with `python -m dapple_amd.build` "
                          "(there is no CPU fallback)" % LIB_PATH)
    # torch first: it ships its own copy of the HIP runtime, and the library's dependency on libamdhip64 must resolve to the
    # copy torch has loaded - a process with two HIP runtimes sees "no ROCm-capable device" in the second one
    import torch  # noqa: F401
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc, what=""):
    if rc != 0:
        msg = load().ds_last_error().decode("utf-8", "replace")
        kind = {-1: ValueError, -2: DappleError, -3: DappleError}.get(rc, DappleError)
        raise kind("%s failed (%d): %s" % (what or "libdapple_hip call", rc, msg))


def profile(on):
    check(load().ds_profile_enable(1 if on else 0), "ds_profile_enable")


def profile_dump():
    """{tag: (launches, total_ms, total_work, unit)} of the launches since the last dump."""
    buf = C.create_string_buffer(1 << 16)
    check(load().ds_profile_dump(buf, len(buf)), "ds_profile_dump")
    out = {}
    for line in buf.value.decode().splitlines():
        tag, n, ms, work, unit = line.split("\t")
        out[tag] = (int(n), float(ms), float(work), unit)
    return out


def ptr(t):
    """Device pointer of a torch tensor (or None)."""
    return None if t is None else C.c_void_p(t.data_ptr())


def current_stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)
