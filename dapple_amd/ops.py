"""Torch-tensor front ends of the per-kernel C-ABI entry points.

Each function takes CUDA (ROCm) tensors, passes raw device pointers through
ctypes and launches on torch's current stream.  Nothing here computes on the
host and nothing falls back to torch ops.
"""
import ctypes as C
import math

import torch

from . import _lib
from ._lib import (DS_BF16, DS_EPI_ACCUM, DS_EPI_BIAS, DS_EPI_DGELU, DS_EPI_GELU, DS_EPI_OUT_F32,
                   DS_EPI_RELU, DS_EPI_RESIDUAL, DS_F32, DS_K_MAJOR, DS_MN_MAJOR, GemmDesc, check, ptr)


def dtype_code(t):
    if t.dtype == torch.float32:
        return DS_F32
    if t.dtype == torch.bfloat16:
        return DS_BF16
    raise ValueError("unsupported element type %s (fp32 or bf16)" % t.dtype)


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("tensor must live on the GPU")
        if t is not None and not t.is_contiguous():
            raise ValueError("tensor must be contiguous")


def _expect(what, t, dtype, shape):
    """``t`` (None allowed) must have exactly this element type and shape: the kernels index by these sizes unchecked."""
    if t is None:
        return
    if t.dtype != dtype or tuple(t.shape) != tuple(shape):
        raise ValueError("%s must be %s %s, got %s %s" % (what, dtype, list(shape), t.dtype, list(t.shape)))


def grad_accumulate(acc, g):
    """acc (fp32) += g, in place (tf.accumulate_n of bert/graph.py:159, one micro-batch at a time)."""
    _need_cuda(acc, g)
    if acc.dtype != torch.float32 or acc.numel() != g.numel():
        raise ValueError("acc must be fp32 with as many elements as g")
    check(_lib.load().ds_grad_accumulate(ptr(acc), ptr(g), g.numel(), dtype_code(g), _lib.current_stream()),
          "ds_grad_accumulate")
    return acc


def cast_to_bf16(src):
    _need_cuda(src)
    dst = torch.empty_like(src, dtype=torch.bfloat16)
    check(_lib.load().ds_cast_f32_to_bf16(ptr(dst), ptr(src), src.numel(), _lib.current_stream()), "ds_cast_f32_to_bf16")
    return dst


def cast_to_f32(src):
    _need_cuda(src)
    dst = torch.empty_like(src, dtype=torch.float32)
    check(_lib.load().ds_cast_bf16_to_f32(ptr(dst), ptr(src), src.numel(), _lib.current_stream()), "ds_cast_bf16_to_f32")
    return dst


def _check_gemm_operands(a, b, c, m, n, k, a_major, b_major, lda, ldb, ldc, flags, batch, a_strides, b_strides, c_strides,
                         bias, residual, c2, k_segment=0, a_segment_stride=0, b_segment_stride=0, batch_inner=1):
    """Every element the kernels may touch must lie inside the tensors handed in: a wrong shape would fault the GPU."""
    if a.dtype != b.dtype:
        raise ValueError("A and B must have one element type")
    want_c = torch.float32 if (flags & (DS_EPI_OUT_F32 | DS_EPI_ACCUM)) or a.dtype == torch.float32 else torch.bfloat16
    if c.dtype != want_c:
        raise ValueError("C must be %s for these flags" % want_c)
    inner = max(batch_inner, 1)
    if batch % inner:
        raise ValueError("batch must be a multiple of batch_inner")

    def extent(rows, cols, ld, strides):   # batch entry z sits at (z // inner) * strides[0] + (z % inner) * strides[1]
        return (rows - 1) * ld + cols + (batch // inner - 1) * abs(strides[0]) + (inner - 1) * abs(strides[1])
    if k_segment:
        if (a_major != DS_MN_MAJOR and b_major != DS_MN_MAJOR) or k_segment <= 0 or k % k_segment or a_segment_stride < 0 or b_segment_stride < 0:
            raise ValueError("a segmented reduction needs an MN-major operand, k_segment dividing k and non-negative segment strides")
        nseg = k // k_segment
        need_a = extent(m, k, lda, a_strides) if a_major == DS_K_MAJOR else extent(k_segment, m, lda, a_strides) + (nseg - 1) * a_segment_stride
        need_b = extent(n, k, ldb, b_strides) if b_major == DS_K_MAJOR else extent(k_segment, n, ldb, b_strides) + (nseg - 1) * b_segment_stride
    else:
        need_a = extent(m, k, lda, a_strides) if a_major == DS_K_MAJOR else extent(k, m, lda, a_strides)
        need_b = extent(n, k, ldb, b_strides) if b_major == DS_K_MAJOR else extent(k, n, ldb, b_strides)
    need_c = extent(m, n, ldc, c_strides)
    if a.numel() < need_a or b.numel() < need_b or c.numel() < need_c:
        raise ValueError("operand too small: A %d < %d, B %d < %d or C %d < %d elements" %
                         (a.numel(), need_a, b.numel(), need_b, c.numel(), need_c))
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() < n):
        raise ValueError("bias must be fp32 with at least n elements")
    if residual is not None and residual.numel() < need_c:
        raise ValueError("residual too small")
    if c2 is not None and c2.numel() < need_c:
        raise ValueError("c2 too small")


def _gemm_desc(a, b, c, m, n, k, a_major, b_major, lda, ldb, ldc, flags, alpha, bias, residual, c2, batch, batch_inner,
               a_strides, b_strides, c_strides, k_segment=0, a_segment_stride=0, b_segment_stride=0):
    _need_cuda(a, b, c, bias, residual, c2)
    d = GemmDesc()
    d.dtype = dtype_code(a)
    d.a_major, d.b_major = a_major, b_major
    d.m, d.n, d.k = m, n, k
    d.lda = lda if lda is not None else (k if a_major == DS_K_MAJOR else m)
    d.ldb = ldb if ldb is not None else (k if b_major == DS_K_MAJOR else n)
    d.ldc = ldc if ldc is not None else n
    _check_gemm_operands(a, b, c, m, n, k, a_major, b_major, d.lda, d.ldb, d.ldc, flags, batch, a_strides, b_strides,
                         c_strides, bias, residual, c2, k_segment, a_segment_stride, b_segment_stride, batch_inner)
    d.k_segment, d.a_segment_stride, d.b_segment_stride = k_segment, a_segment_stride, b_segment_stride
    d.batch, d.batch_inner = batch, batch_inner
    d.a_stride_outer, d.a_stride_inner = a_strides
    d.b_stride_outer, d.b_stride_inner = b_strides
    d.c_stride_outer, d.c_stride_inner = c_strides
    d.flags, d.alpha = flags, alpha
    d.a, d.b, d.c = a.data_ptr(), b.data_ptr(), c.data_ptr()
    d.bias = bias.data_ptr() if bias is not None else None
    d.residual = residual.data_ptr() if residual is not None else None
    d.c2 = c2.data_ptr() if c2 is not None else None
    return d


def gemm_grouped(problems):
    """ds_gemm_grouped: `problems` is a list of dicts with the keyword arguments of `gemm` (a, b, c, m, n, k, a_major,
    b_major, flags, bias, residual, c2, ...) plus `cfg`, the tile shape (0 = 256x256, 1 = 256x128, 2 = 128x128,
    3 = 128x64); all of them run as one launch, workgroups starting in list order."""
    n = len(problems)
    descs = (GemmDesc * n)()
    cfgs = (C.c_int * n)()
    for i, p in enumerate(problems):
        p = dict(p)
        cfgs[i] = p.pop("cfg", 2)
        args = dict(a_major=DS_K_MAJOR, b_major=DS_MN_MAJOR, lda=None, ldb=None, ldc=None, flags=0, alpha=1.0, bias=None,
                    residual=None, c2=None, batch=1, batch_inner=1, a_strides=(0, 0), b_strides=(0, 0), c_strides=(0, 0))
        args.update(p)
        descs[i] = _gemm_desc(**args)
    check(_lib.load().ds_gemm_grouped(descs, cfgs, n, _lib.current_stream()), "ds_gemm_grouped")


def gemm(a, b, c, m, n, k, a_major=DS_K_MAJOR, b_major=DS_MN_MAJOR, lda=None, ldb=None, ldc=None, flags=0,
         alpha=1.0, bias=None, residual=None, c2=None, batch=1, batch_inner=1, a_strides=(0, 0), b_strides=(0, 0),
         c_strides=(0, 0), workspace=None, static_scratch=False, k_segment=0, a_segment_stride=0, b_segment_stride=0):
    """Raw ds_gemm: C[m][n] (+)= alpha * sum_k A(m,k) B(n,k); see include/dapple_stage.h.  `workspace`: a zero-filled
    uint8 tensor of gemm_workspace_bytes(m, n) bytes that lets the library cut a long k into slices (split-K);
    `static_scratch`: ds_gemm_static_scratch instead, the variant that allocates nothing (the library's own scratch).
    `k_segment` (MN-major operands): the reduction runs over k / k_segment segments whose first rows are
    `a_segment_stride` / `b_segment_stride` elements apart."""
    _need_cuda(workspace)
    d = _gemm_desc(a, b, c, m, n, k, a_major, b_major, lda, ldb, ldc, flags, alpha, bias, residual, c2, batch, batch_inner,
                   a_strides, b_strides, c_strides, k_segment, a_segment_stride, b_segment_stride)
    if workspace is not None:
        d.workspace, d.workspace_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    if static_scratch:
        check(_lib.load().ds_gemm_static_scratch(C.byref(d), _lib.current_stream()), "ds_gemm_static_scratch")
    else:
        check(_lib.load().ds_gemm(C.byref(d), _lib.current_stream()), "ds_gemm")


def gemm_workspace_bytes(m, n):
    """Bytes of split-K workspace ds_gemm wants for an [m, n] output (zero-fill it once before the first use)."""
    return int(_lib.load().ds_gemm_workspace_bytes(m, n))


def dense(x, kernel, bias=None, residual=None, gelu=False):
    """tf.layers.dense: x[m,k] @ kernel[k,n] + bias (+ residual) (gelu -> returns (pre, act))."""
    m, k = x.shape
    n = kernel.shape[1]
    y = torch.empty(m, n, dtype=x.dtype, device=x.device)
    flags = (DS_EPI_BIAS if bias is not None else 0) | (DS_EPI_RESIDUAL if residual is not None else 0)
    act = None
    if gelu:
        flags |= DS_EPI_GELU
        act = torch.empty_like(y)
    gemm(x, kernel, y, m, n, k, DS_K_MAJOR, DS_MN_MAJOR, flags=flags, bias=bias, residual=residual, c2=act)
    return (y, act) if gelu else y


def layernorm_fwd(x, gamma, beta, eps=1e-12):
    _need_cuda(x, gamma, beta)
    rows, cols = x.shape
    y = torch.empty_like(x)
    stats = torch.empty(rows, 2, dtype=torch.float32, device=x.device)
    check(_lib.load().ds_layernorm_fwd(dtype_code(x), rows, cols, ptr(x), ptr(gamma), ptr(beta), eps, ptr(y), ptr(stats),
                                       _lib.current_stream()), "ds_layernorm_fwd")
    return y, stats


def layernorm_bwd(dy, x, gamma, stats, d_gamma, d_beta, d_colsum=None, dx_add=None):
    _need_cuda(dy, x, gamma, stats, d_gamma, d_beta, d_colsum, dx_add)
    rows, cols = x.shape
    dx = torch.empty_like(x)
    check(_lib.load().ds_layernorm_bwd(dtype_code(x), rows, cols, ptr(dy), ptr(x), ptr(gamma), ptr(stats), ptr(dx_add),
                                       ptr(dx), ptr(d_gamma), ptr(d_beta), ptr(d_colsum), _lib.current_stream()),
          "ds_layernorm_bwd")
    return dx


def layernorm_fwd_mixed(x, gamma, beta, eps=1e-12, want_f32=True):
    """LayerNorm on an fp32 residual stream: x fp32 -> (y bf16, y fp32 or None, stats)."""
    _need_cuda(x, gamma, beta)
    if x.dtype != torch.float32:
        raise ValueError("layernorm_fwd_mixed: x must be fp32")
    rows, cols = x.shape
    y16 = torch.empty(rows, cols, dtype=torch.bfloat16, device=x.device)
    y32 = torch.empty_like(x) if want_f32 else None
    stats = torch.empty(rows, 2, dtype=torch.float32, device=x.device)
    check(_lib.load().ds_layernorm_fwd_mixed(rows, cols, ptr(x), ptr(gamma), ptr(beta), eps, ptr(y16), ptr(y32), ptr(stats),
                                             _lib.current_stream()), "ds_layernorm_fwd_mixed")
    return y16, y32, stats


def layernorm_bwd_mixed(dy, x, gamma, stats, d_gamma=None, d_beta=None, d_colsum=None, want_f32=True, want_dy_bf16=False):
    """Backward of ``layernorm_fwd_mixed``: dy, x fp32 -> (dx bf16, dx fp32 or None); parameter gradients are added to.
    Without ``d_gamma`` / ``d_beta`` only dx is computed (no atomics); ``want_dy_bf16`` then also returns the bf16 copy of
    dy that ``layernorm_param_grads_mixed`` takes: (dx bf16, dx fp32 or None, dy bf16)."""
    _need_cuda(dy, x, gamma, stats, d_gamma, d_beta, d_colsum)
    rows, cols = _check_ln_mixed(x, gamma, stats, [(dy, torch.float32)])
    for t in (d_gamma, d_beta, d_colsum):
        if t is not None and (t.dtype != torch.float32 or t.numel() != cols):
            raise ValueError("parameter gradients must be fp32 [cols]")
    dx16 = torch.empty(rows, cols, dtype=torch.bfloat16, device=x.device)
    dx32 = torch.empty_like(x) if want_f32 else None
    dy16 = torch.empty_like(dx16) if want_dy_bf16 else None
    check(_lib.load().ds_layernorm_bwd_mixed(rows, cols, ptr(dy), ptr(x), ptr(gamma), ptr(stats), ptr(dx16), ptr(dx32), ptr(dy16),
                                             ptr(d_gamma), ptr(d_beta), ptr(d_colsum), _lib.current_stream()), "ds_layernorm_bwd_mixed")
    return (dx16, dx32, dy16) if want_dy_bf16 else (dx16, dx32)


def _check_ln_mixed(x, gamma, stats, others=()):
    """The row kernels index every tensor by x's shape: anything smaller is read or written out of bounds."""
    if x.dim() != 2 or x.dtype != torch.float32:
        raise ValueError("x must be a 2-D fp32 tensor")
    rows, cols = x.shape
    if gamma.dtype != torch.float32 or gamma.numel() != cols or stats.dtype != torch.float32 or stats.numel() != 2 * rows:
        raise ValueError("gamma must be fp32 [cols] and stats fp32 [rows, 2]")
    for t, dt in others:
        if t is not None and (t.dtype != dt or t.numel() != rows * cols):
            raise ValueError("tensor of %s with x's shape expected" % dt)
    return rows, cols


def layernorm_bwd_mixed_rows(dy, x, gamma, stats, want_f32=True):
    """ds_layernorm_bwd_mixed_rows: dy, x fp32 -> (dx bf16, dx fp32 or None, fp32 copy of dy, per-row means [rows, 2])."""
    _need_cuda(dy, x, gamma, stats)
    rows, cols = _check_ln_mixed(x, gamma, stats, [(dy, torch.float32)])
    dx16 = torch.empty(rows, cols, dtype=torch.bfloat16, device=x.device)
    dx32 = torch.empty_like(x) if want_f32 else None
    dyc = torch.empty_like(x)
    row_sums = torch.empty(rows, 2, dtype=torch.float32, device=x.device)
    check(_lib.load().ds_layernorm_bwd_mixed_rows(rows, cols, ptr(dy), ptr(x), ptr(gamma), ptr(stats), ptr(dx16), ptr(dx32), ptr(dyc),
                                                  ptr(row_sums), _lib.current_stream()), "ds_layernorm_bwd_mixed_rows")
    return dx16, dx32, dyc, row_sums


def layernorm_param_grads_exact(dy_copy, x, gamma, stats, row_sums, d_gamma, d_beta, d_colsum=None):
    """ds_layernorm_param_grads_exact: the deferred half of ``layernorm_bwd_mixed_rows``, without rounding."""
    _need_cuda(dy_copy, x, gamma, stats, row_sums, d_gamma, d_beta, d_colsum)
    rows, cols = _check_ln_mixed(x, gamma, stats, [(dy_copy, torch.float32)])
    if row_sums.dtype != torch.float32 or row_sums.numel() != 2 * rows:
        raise ValueError("row_sums must be fp32 [rows, 2]")
    for t in (d_gamma, d_beta, d_colsum):
        if t is not None and (t.dtype != torch.float32 or t.numel() != cols):
            raise ValueError("parameter gradients must be fp32 [cols]")
    check(_lib.load().ds_layernorm_param_grads_exact(rows, cols, ptr(dy_copy), ptr(x), ptr(gamma), ptr(stats), ptr(row_sums), ptr(d_gamma),
                                                     ptr(d_beta), ptr(d_colsum), _lib.current_stream()), "ds_layernorm_param_grads_exact")


def layernorm_param_grads_mixed(dy_bf16, x, stats, d_gamma, d_beta, dx_bf16=None, d_colsum=None):
    """d_gamma += sum_rows dy * x_hat, d_beta += sum_rows dy, d_colsum += sum_rows dx from the bf16 copies that
    ``layernorm_bwd_mixed(..., want_dy_bf16=True)`` left and the fp32 x: the deferred half of that backward pass."""
    _need_cuda(dy_bf16, x, stats, d_gamma, d_beta, dx_bf16, d_colsum)
    if x.dim() != 2 or x.dtype != torch.float32 or stats.numel() != 2 * x.shape[0]:
        raise ValueError("x must be 2-D fp32 and stats [rows, 2]")
    rows, cols = x.shape
    for t in (dy_bf16, dx_bf16):
        if t is not None and (t.dtype != torch.bfloat16 or t.numel() != rows * cols):
            raise ValueError("dy_bf16 / dx_bf16 must be bf16 with x's shape")
    for t in (d_gamma, d_beta, d_colsum):
        if t is not None and (t.dtype != torch.float32 or t.numel() != cols):
            raise ValueError("parameter gradients must be fp32 [cols]")
    check(_lib.load().ds_layernorm_param_grads_mixed(rows, cols, ptr(dy_bf16), ptr(x), ptr(stats), ptr(dx_bf16), ptr(d_gamma),
                                                     ptr(d_beta), ptr(d_colsum), _lib.current_stream()),
          "ds_layernorm_param_grads_mixed")


def layernorm_param_grads(dy, x, stats, d_gamma, d_beta, dx=None, d_colsum=None):
    """d_gamma += sum_rows dy * x_hat, d_beta += sum_rows dy, d_colsum += sum_rows dx: the half of the LayerNorm backward
    pass that ``layernorm_bwd(..., d_gamma=None, d_beta=None)`` leaves out."""
    _need_cuda(dy, x, stats, d_gamma, d_beta, dx, d_colsum)
    rows, cols = x.shape
    check(_lib.load().ds_layernorm_param_grads(dtype_code(x), rows, cols, ptr(dy), ptr(x), ptr(stats), ptr(dx), ptr(d_gamma),
                                               ptr(d_beta), ptr(d_colsum), _lib.current_stream()), "ds_layernorm_param_grads")


def softmax_fwd(scores, scale, key_mask=None, mask_value=-10000.0, out_dtype=torch.float32):
    """scores fp32 [B, N, Q, K] -> probabilities of out_dtype."""
    _need_cuda(scores, key_mask)
    b, n, q, k = scores.shape
    if scores.dtype != torch.float32 or out_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("softmax_fwd: fp32 scores, fp32 or bf16 probabilities")
    _expect("softmax_fwd: key_mask", key_mask, torch.float32, (b, k))
    p = torch.empty(b, n, q, k, dtype=out_dtype, device=scores.device)
    check(_lib.load().ds_softmax_fwd(dtype_code(p), b, n, q, k, ptr(scores), scale, ptr(key_mask), mask_value, ptr(p),
                                     _lib.current_stream()), "ds_softmax_fwd")
    return p


def softmax_bwd(p, dp, scale):
    _need_cuda(p, dp)
    if dp.dtype != torch.float32 or dp.shape != p.shape:
        raise ValueError("softmax_bwd: dp must be fp32 with the shape of p")
    k = p.shape[-1]
    rows = p.numel() // k
    ds = torch.empty_like(p)
    check(_lib.load().ds_softmax_bwd(dtype_code(p), rows, k, ptr(p), ptr(dp), scale, ptr(ds), _lib.current_stream()),
          "ds_softmax_bwd")
    return ds


def colsum_accum(x, out):
    _need_cuda(x, out)
    rows, cols = x.shape
    _expect("colsum_accum: out", out, torch.float32, (cols,))
    check(_lib.load().ds_colsum_accum(dtype_code(x), rows, cols, ptr(x), cols, ptr(out), _lib.current_stream()),
          "ds_colsum_accum")
    return out


def conv3x3(x, kernel, bias=None, relu=False, mask_src=None):
    """NHWC fp32 3x3 'same' convolution (keras Conv2D of vgg19_slice_model.py:137); kernel HWIO."""
    _need_cuda(x, kernel, bias, mask_src)
    n, h, w, cin = x.shape
    cout = kernel.shape[-1]
    y = torch.empty(n, h, w, cout, dtype=x.dtype, device=x.device)
    flags = (DS_EPI_BIAS if bias is not None else 0) | (DS_EPI_RELU if relu else 0) | (128 if mask_src is not None else 0)
    check(_lib.load().ds_conv3x3_fwd(dtype_code(x), n, h, w, cin, cout, ptr(x), ptr(kernel), ptr(bias), flags, ptr(mask_src),
                                     ptr(y), _lib.current_stream()), "ds_conv3x3_fwd")
    return y


def conv3x3_wgrad(x, dz, dkernel):
    """dkernel (HWIO fp32) += correlation of x with dz."""
    _need_cuda(x, dz, dkernel)
    n, h, w, cin = x.shape
    cout = dz.shape[-1]
    check(_lib.load().ds_conv3x3_wgrad(dtype_code(x), n, h, w, cin, cout, ptr(x), ptr(dz), ptr(dkernel),
                                       _lib.current_stream()), "ds_conv3x3_wgrad")
    return dkernel


def conv3x3_flip(kernel):
    _need_cuda(kernel)
    cin, cout = kernel.shape[2], kernel.shape[3]
    out = torch.empty(3, 3, cout, cin, dtype=torch.float32, device=kernel.device)
    check(_lib.load().ds_conv3x3_flip(cin, cout, ptr(kernel), ptr(out), _lib.current_stream()), "ds_conv3x3_flip")
    return out


def maxpool2x2(x):
    _need_cuda(x)
    n, h, w, c = x.shape
    y = torch.empty(n, h // 2, w // 2, c, dtype=x.dtype, device=x.device)
    check(_lib.load().ds_maxpool2x2_fwd(n, h, w, c, ptr(x), ptr(y), _lib.current_stream()), "ds_maxpool2x2_fwd")
    return y


def maxpool2x2_bwd(x, dy, relu_mask=False):
    _need_cuda(x, dy)
    n, h, w, c = x.shape
    dx = torch.empty_like(x)
    check(_lib.load().ds_maxpool2x2_bwd(n, h, w, c, ptr(x), ptr(dy), ptr(dx), 1 if relu_mask else 0, _lib.current_stream()),
          "ds_maxpool2x2_bwd")
    return dx


def attention_fwd(qkv, batch, heads, seq, scale, key_mask=None, mask_value=-10000.0):
    """Fused bf16 attention on the fused projection qkv [batch*seq, 3*heads*64] -> (ctx, lse)."""
    _need_cuda(qkv, key_mask)
    _check_attention(qkv, batch, heads, seq, key_mask=key_mask)
    hidden = qkv.shape[1] // 3
    ctx = torch.empty(batch * seq, hidden, dtype=qkv.dtype, device=qkv.device)
    lse = torch.empty(batch, heads, seq, dtype=torch.float32, device=qkv.device)
    check(_lib.load().ds_attention_fwd(dtype_code(qkv), batch, heads, seq, hidden // heads, ptr(qkv), qkv.shape[1], ptr(key_mask),
                                       scale, mask_value, ptr(ctx), ptr(lse), _lib.current_stream()), "ds_attention_fwd")
    return ctx, lse


def _check_attention(qkv, batch, heads, seq, others=(), key_mask=None):
    """Shapes the fused attention kernels index by: a wrong one reads or writes outside the tensors."""
    if qkv.dim() != 2 or qkv.shape[0] != batch * seq or qkv.shape[1] % (3 * heads) != 0:
        raise ValueError("qkv must be [batch * seq, 3 * heads * head_size]")
    for t in others:
        if t.dtype != qkv.dtype or tuple(t.shape) != (batch * seq, qkv.shape[1] // 3):
            raise ValueError("ctx / dctx must be [batch * seq, heads * head_size] of qkv's element type")
    if key_mask is not None and (key_mask.dtype != torch.float32 or key_mask.numel() != batch * seq):
        raise ValueError("key_mask must be fp32 [batch, seq]")


def attention_key_mean(qkv, batch, heads, seq):
    """Mean key of every sample and head, fp32 [batch, heads * 64] (ds_attention_key_mean)."""
    _need_cuda(qkv)
    _check_attention(qkv, batch, heads, seq)
    hidden = qkv.shape[1] // 3
    out = torch.empty(batch, hidden, dtype=torch.float32, device=qkv.device)
    check(_lib.load().ds_attention_key_mean(dtype_code(qkv), batch, heads, seq, hidden // heads, ptr(qkv), qkv.shape[1], ptr(out), _lib.current_stream()),
          "ds_attention_key_mean")
    return out


def attention_bwd(qkv, ctx, lse, dctx, batch, heads, seq, scale, key_mask=None, mask_value=-10000.0, key_mean=None):
    """``key_mean`` (from ``attention_key_mean``): ds_attention_bwd_centered, which keeps the rounding of the score gradients
    out of dq."""
    _need_cuda(qkv, ctx, lse, dctx, key_mask, key_mean)
    _check_attention(qkv, batch, heads, seq, (ctx, dctx), key_mask)
    if lse.dtype != torch.float32 or lse.numel() != batch * heads * seq:
        raise ValueError("lse must be fp32 [batch, heads, seq]")
    if key_mean is not None and (key_mean.dtype != torch.float32 or key_mean.numel() != batch * (qkv.shape[1] // 3)):
        raise ValueError("key_mean must be fp32 [batch, heads * head_size]")
    hidden = qkv.shape[1] // 3
    dqkv = torch.empty_like(qkv)
    delta = torch.empty_like(lse)
    check(_lib.load().ds_attention_bwd_centered(dtype_code(qkv), batch, heads, seq, hidden // heads, ptr(qkv), qkv.shape[1],
                                                ptr(key_mask), scale, mask_value, ptr(ctx), ptr(lse), ptr(dctx), ptr(dqkv), ptr(delta),
                                                ptr(key_mean), _lib.current_stream()), "ds_attention_bwd")
    return dqkv


def xlnet_scores_pack(seq, rows, klen, batch, masks=None, seg_mat=None):
    """Mask (fp32 [rows, klen, batch], non-zero = masked) and segment matrix (uint8 [seq, klen, batch]) as the packed bits
    ``xlnet_scores_fwd`` / ``xlnet_scores_bwd`` read -> (meta, nseg); (None, None) when both are None."""
    if masks is None and seg_mat is None:
        return None, None
    _need_cuda(masks, seg_mat)
    _expect("xlnet_scores_pack: masks", masks, torch.float32, (rows, klen, batch))
    _expect("xlnet_scores_pack: seg_mat", seg_mat, torch.uint8, (seq, klen, batch))
    if rows % seq:
        raise ValueError("xlnet_scores_pack: rows must be a multiple of seq (the streams are stacked)")
    lib = _lib.load()
    dev = (masks if masks is not None else seg_mat).device
    meta = torch.empty(lib.ds_xlnet_scores_meta_bytes(rows, klen, batch), dtype=torch.uint8, device=dev)
    nseg = torch.zeros(batch, seq, dtype=torch.float32, device=dev) if seg_mat is not None else None
    check(lib.ds_xlnet_scores_pack(seq, rows, klen, batch, ptr(masks), ptr(seg_mat), ptr(meta), ptr(nseg), _lib.current_stream()),
          "ds_xlnet_scores_pack")
    return meta, nseg


def xlnet_bias_q(q, bias_context, bias_relative, bias_segment, seg_emb, heads):
    """``q [rows, batch, H]`` (bf16) -> (qw, qr, qs, de): q plus the three relative-attention biases (fp32 ``[H]``) and
    ``de [batch, heads, rows]`` = qs . (seg_emb[1] - seg_emb[0]) per head."""
    _need_cuda(q, bias_context, bias_relative, bias_segment, seg_emb)
    rows, batch, hidden = q.shape
    if q.dtype != torch.bfloat16 or hidden != heads * 64:
        raise ValueError("xlnet_bias_q: q must be bf16 [rows, batch, heads * 64]")
    for name, t in (("bias_context", bias_context), ("bias_relative", bias_relative), ("bias_segment", bias_segment)):
        if t.dtype != torch.float32 or t.numel() != hidden:
            raise ValueError("xlnet_bias_q: %s must be fp32 with heads * 64 elements" % name)
    if seg_emb.dtype != torch.float32 or seg_emb.numel() != 2 * hidden:
        raise ValueError("xlnet_bias_q: seg_emb must be fp32 [2, heads, 64]")
    qw, qr, qs = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    de = torch.empty(batch, heads, rows, dtype=torch.float32, device=q.device)
    check(_lib.load().ds_xlnet_bias_q(rows, batch, heads, ptr(q), ptr(bias_context), ptr(bias_relative), ptr(bias_segment), ptr(seg_emb),
                                      ptr(qw), ptr(qr), ptr(qs), ptr(de), _lib.current_stream()), "ds_xlnet_bias_q")
    return qw, qr, qs, de


def _xlnet_scores_check(what, seq, rows, klen, batch, heads, hidden, kv, meta):
    if hidden != heads * 64 or rows % seq or klen < seq:
        raise ValueError("%s: head size 64, rows a multiple of seq and klen >= seq are required" % what)
    _expect(what + ": kv", kv, torch.bfloat16, (klen, batch, 2 * hidden))
    if meta is not None and (meta.dtype != torch.uint8 or meta.numel() != _lib.load().ds_xlnet_scores_meta_bytes(rows, klen, batch)):
        raise ValueError("%s: meta must be what xlnet_scores_pack returned for these sizes" % what)


def xlnet_scores_fwd(qw, qr, de, kv, kr, seq, heads, scale, meta=None):
    """Probabilities of XLNet's relative attention (bf16, head size 64): ``qw, qr [rows, batch, H]`` and ``de`` from
    ``xlnet_bias_q``, ``kv [klen, batch, 2H]``, ``kr [klen + seq, H]`` -> ``p [batch*heads, rows, klen]``."""
    _need_cuda(qw, qr, de, kv, kr, meta)
    rows, batch, hidden = qw.shape
    klen = kv.shape[0]
    _xlnet_scores_check("xlnet_scores_fwd", seq, rows, klen, batch, heads, hidden, kv, meta)
    _expect("xlnet_scores_fwd: qw", qw, torch.bfloat16, (rows, batch, hidden))
    _expect("xlnet_scores_fwd: qr", qr, torch.bfloat16, (rows, batch, hidden))
    _expect("xlnet_scores_fwd: de", de, torch.float32, (batch, heads, rows))
    _expect("xlnet_scores_fwd: kr", kr, torch.bfloat16, (klen + seq, hidden))
    p = torch.empty(batch * heads, rows, klen, dtype=qw.dtype, device=qw.device)
    check(_lib.load().ds_xlnet_scores_fwd(seq, rows, klen, batch, heads, ptr(qw), ptr(qr), ptr(de), ptr(kv), ptr(kr), ptr(meta), scale,
                                          ptr(p), _lib.current_stream()), "ds_xlnet_scores_fwd")
    return p


def xlnet_scores_bwd(kv, p, dvec, seq, heads, scale, meta=None, nseg=None, dbd=None):
    """Score gradients of the same rows from ``dvec [rows, batch, H]`` (gradient of ``p v``): -> (ds, dbd, defs); ``dbd``
    ``[batch*heads, rows, klen + seq]`` is written only inside its band (pass a cleared buffer to reuse it)."""
    _need_cuda(kv, p, dvec, meta, nseg, dbd)
    rows, batch, hidden = dvec.shape
    klen = kv.shape[0]
    _xlnet_scores_check("xlnet_scores_bwd", seq, rows, klen, batch, heads, hidden, kv, meta)
    _expect("xlnet_scores_bwd: dvec", dvec, torch.bfloat16, (rows, batch, hidden))
    _expect("xlnet_scores_bwd: p", p, torch.bfloat16, (batch * heads, rows, klen))
    _expect("xlnet_scores_bwd: nseg", nseg, torch.float32, (batch, seq))
    _expect("xlnet_scores_bwd: dbd", dbd, torch.bfloat16, (batch * heads, rows, klen + seq))
    ds = torch.empty_like(p)
    if dbd is None:
        dbd = torch.zeros(batch * heads, rows, klen + seq, dtype=p.dtype, device=p.device)
    defs = torch.empty(batch * heads, rows, 2, dtype=torch.float32, device=p.device)
    check(_lib.load().ds_xlnet_scores_bwd(seq, rows, klen, batch, heads, ptr(kv), ptr(p), ptr(dvec), ptr(meta), ptr(nseg), scale,
                                          ptr(ds), ptr(dbd), ptr(defs), _lib.current_stream()), "ds_xlnet_scores_bwd")
    return ds, dbd, defs


def squad_head(x, batch, seq, output_weights, output_bias, start_positions, end_positions, d_weights=None, d_bias=None,
               need_dx=True, loss_scale=1.0):
    """build_output_layer_squad of bert/models/bert/bert.py:669-718 on the stage's sequence output
    ``x [batch*seq, hidden]``: returns (loss [1] fp32 on the device, start_logits [batch, seq], end_logits
    [batch, seq], dx or None).  ``d_weights [2, hidden]`` / ``d_bias [2]`` (fp32) are added to in place."""
    _need_cuda(x, output_weights, output_bias, start_positions, end_positions)
    hidden = x.shape[-1]
    if x.numel() != batch * seq * hidden or tuple(output_weights.shape) != (2, hidden):
        raise ValueError("squad_head: x must be [batch*seq, hidden] and output_weights [2, hidden]")
    if start_positions.dtype != torch.int32 or end_positions.dtype != torch.int32:
        raise ValueError("squad_head: positions must be int32")
    for t in (output_weights, output_bias, d_weights, d_bias):
        if t is not None and t.dtype != torch.float32:
            raise ValueError("squad_head: weights, bias and their gradients must be fp32")
    loss = torch.empty(1, dtype=torch.float32, device=x.device)
    logits = torch.empty(batch * seq, 2, dtype=torch.float32, device=x.device)
    dlogits = torch.empty_like(logits)
    dx = torch.empty_like(x) if need_dx else None
    check(_lib.load().ds_squad_head(dtype_code(x), batch, seq, hidden, ptr(x), ptr(output_weights), ptr(output_bias),
                                    ptr(start_positions), ptr(end_positions), loss_scale, ptr(loss), ptr(logits), ptr(dlogits),
                                    ptr(dx), ptr(d_weights), ptr(d_bias), _lib.current_stream()), "ds_squad_head")
    lg = logits.view(batch, seq, 2)
    return loss, lg[:, :, 0], lg[:, :, 1], dx


def pooler(x, batch, seq, pooler_w, pooler_b):
    """pooler_stage (modeling_slice.py:849-868): tanh dense on each sample's first token -> fp32 [batch, hidden]."""
    _need_cuda(x, pooler_w, pooler_b)
    hidden = pooler_w.shape[1]
    if x.numel() != batch * seq * hidden or tuple(pooler_w.shape) != (hidden, hidden) or pooler_b.numel() != hidden:
        raise ValueError("pooler: x must be [batch*seq, hidden], pooler_w [hidden, hidden], pooler_b [hidden]")
    if pooler_w.dtype != torch.float32 or pooler_b.dtype != torch.float32:
        raise ValueError("pooler: the dense parameters are fp32")
    pooled = torch.empty(batch, hidden, dtype=torch.float32, device=x.device)
    check(_lib.load().ds_pooler(dtype_code(x), batch, seq, hidden, ptr(x), ptr(pooler_w), ptr(pooler_b), ptr(pooled),
                                _lib.current_stream()), "ds_pooler")
    return pooled


def lstm_cell_fwd(gates, c_prev=None, forget_bias=1.0, x_residual=None):
    """One BasicLSTMCell step on pre-activations ``gates`` fp32 [batch, 4*units] (overwritten with the activated gates):
    returns (c, h, y) with y = h + x_residual or None."""
    _need_cuda(gates, c_prev, x_residual)
    b, u4 = gates.shape
    u = u4 // 4
    if gates.dtype != torch.float32 or u4 != 4 * u or u == 0:
        raise ValueError("lstm_cell_fwd: gates must be fp32 [batch, 4 * units]")
    _expect("lstm_cell_fwd: c_prev", c_prev, torch.float32, (b, u))
    _expect("lstm_cell_fwd: x_residual", x_residual, torch.float32, (b, u))
    c = torch.empty(b, u, dtype=torch.float32, device=gates.device)
    h = torch.empty_like(c)
    y = torch.empty_like(c) if x_residual is not None else None
    check(_lib.load().ds_lstm_cell_fwd(b, u, forget_bias, ptr(gates), ptr(c_prev), ptr(c), ptr(h), ptr(x_residual), ptr(y),
                                       _lib.current_stream()), "ds_lstm_cell_fwd")
    return c, h, y


def lstm_cell_bwd(gates_act, c, c_prev, dh, dc, first):
    """Backward of one BasicLSTMCell step: returns dgates [batch, 4*units]; ``dc`` [batch, units] carries the cell-state
    gradient between steps (read unless ``first``, then overwritten with dc * f)."""
    _need_cuda(gates_act, c, c_prev, dh, dc)
    b, u4 = gates_act.shape
    u = u4 // 4
    if gates_act.dtype != torch.float32 or u4 != 4 * u or u == 0:
        raise ValueError("lstm_cell_bwd: gates_act must be fp32 [batch, 4 * units]")
    for name, t in (("c", c), ("c_prev", c_prev), ("dh", dh), ("dc", dc)):
        _expect("lstm_cell_bwd: " + name, t, torch.float32, (b, u))
    if c is None or dh is None or dc is None:
        raise ValueError("lstm_cell_bwd: c, dh and dc are required")
    dgates = torch.empty_like(gates_act)
    check(_lib.load().ds_lstm_cell_bwd(b, u4 // 4, ptr(gates_act), ptr(c), ptr(c_prev), ptr(dh), ptr(dc), 1 if first else 0,
                                       ptr(dgates), _lib.current_stream()), "ds_lstm_cell_bwd")
    return dgates


def classifier_head(x, batch, seq, pooler_w, pooler_b, fc_w, fc_b, labels, grads=None, need_dx=True, l2_scale=1e-3,
                    loss_scale=1.0):
    """pooler_stage (modeling_slice.py:849-868) + build_output_layer_classification (bert.py:642-664) on the stage's
    sequence output ``x [batch*seq, hidden]``: returns (loss [1] fp32 on the device, logits [batch, num_labels], pooled
    [batch, hidden], dx or None).  ``grads`` = (d_pooler_w, d_pooler_b, d_fc_w, d_fc_b), fp32, added to in place."""
    _need_cuda(x, pooler_w, pooler_b, fc_w, fc_b, labels)
    hidden = x.shape[-1]
    if x.numel() != batch * seq * hidden or tuple(pooler_w.shape) != (hidden, hidden) or fc_w.shape[0] != hidden:
        raise ValueError("classifier_head: x must be [batch*seq, hidden], pooler_w [hidden, hidden], fc_w [hidden, num_labels]")
    num_labels = fc_w.shape[1]
    if labels.dtype != torch.int32 or labels.numel() != batch:
        raise ValueError("classifier_head: labels must be int32 [batch]")
    grads = tuple(grads) if grads is not None else (None,) * 4
    for t in (pooler_w, pooler_b, fc_w, fc_b) + grads:
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous()):
            raise ValueError("classifier_head: weights and their gradients must be contiguous fp32")
    f32 = dict(dtype=torch.float32, device=x.device)
    loss, pooled = torch.empty(1, **f32), torch.empty(batch, hidden, **f32)
    logits, dlogits, dz = torch.empty(batch, num_labels, **f32), torch.empty(batch, num_labels, **f32), torch.empty(batch, hidden, **f32)
    dx = torch.empty_like(x) if need_dx else None
    check(_lib.load().ds_classifier_head(dtype_code(x), batch, seq, hidden, num_labels, ptr(x), ptr(pooler_w), ptr(pooler_b), ptr(fc_w),
                                         ptr(fc_b), ptr(labels), l2_scale, loss_scale, ptr(loss), ptr(pooled), ptr(logits), ptr(dlogits),
                                         ptr(dz), ptr(dx), ptr(grads[0]), ptr(grads[1]), ptr(grads[2]), ptr(grads[3]),
                                         _lib.current_stream()), "ds_classifier_head")
    return loss, logits, pooled, dx


def regression_head(x, batch, seq, pooler_w, pooler_b, fc_w, fc_b, targets, grads=None, need_dx=True, l2_scale=1e-3,
                    loss_scale=1.0):
    """pooler_stage (modeling_slice.py:849-868) + build_output_layer_regression (bert.py:615-640) on the stage's sequence
    output ``x [batch*seq, hidden]``; ``targets`` fp32 [batch].  The loss is the reference graph's: the mean over every
    (prediction, label) pair of the squared difference (a [batch, 1] - [batch] broadcast) plus the l2 term.  Returns
    (loss [1] fp32 on the device, prediction [batch, 1], pooled [batch, hidden], dx or None)."""
    _need_cuda(x, pooler_w, pooler_b, fc_w, fc_b, targets)
    hidden = x.shape[-1]
    if x.numel() != batch * seq * hidden or tuple(pooler_w.shape) != (hidden, hidden) or tuple(fc_w.shape) != (hidden, 1):
        raise ValueError("regression_head: x must be [batch*seq, hidden], pooler_w [hidden, hidden], fc_w [hidden, 1]")
    if targets.dtype != torch.float32 or targets.numel() != batch:
        raise ValueError("regression_head: targets must be fp32 [batch]")
    grads = tuple(grads) if grads is not None else (None,) * 4
    for t in (pooler_w, pooler_b, fc_w, fc_b) + grads:
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous()):
            raise ValueError("regression_head: weights and their gradients must be contiguous fp32")
    f32 = dict(dtype=torch.float32, device=x.device)
    loss, pooled = torch.empty(1, **f32), torch.empty(batch, hidden, **f32)
    pred, dpred, dz = torch.empty(batch, 1, **f32), torch.empty(batch, 1, **f32), torch.empty(batch, hidden, **f32)
    dx = torch.empty_like(x) if need_dx else None
    check(_lib.load().ds_regression_head(dtype_code(x), batch, seq, hidden, ptr(x), ptr(pooler_w), ptr(pooler_b), ptr(fc_w), ptr(fc_b),
                                         ptr(targets), l2_scale, loss_scale, ptr(loss), ptr(pooled), ptr(pred), ptr(dpred), ptr(dz),
                                         ptr(dx), ptr(grads[0]), ptr(grads[1]), ptr(grads[2]), ptr(grads[3]),
                                         _lib.current_stream()), "ds_regression_head")
    return loss, pred, pooled, dx


XLNET_HEAD_SHAPES = {"start_w": lambda h: (h,), "start_b": lambda h: (1,), "end_w0": lambda h: (2 * h, h), "end_b0": lambda h: (h,),
                     "ln_gamma": lambda h: (h,), "ln_beta": lambda h: (h,), "end_w1": lambda h: (h,), "end_b1": lambda h: (1,),
                     "ans_w0": lambda h: (2 * h, h), "ans_b0": lambda h: (h,), "ans_w1": lambda h: (h,)}


def _xlnet_head_params(tensors, hidden, what):
    out = _lib.XlnetHeadParams()
    for name in _lib.XLNET_HEAD_TENSORS:
        t = tensors[name]
        if t.dtype != torch.float32 or not t.is_contiguous() or not t.is_cuda or t.numel() != math.prod(XLNET_HEAD_SHAPES[name](hidden)):
            raise ValueError(f"xlnet_squad_head: {what}[{name!r}] must be a contiguous fp32 device tensor of shape "
                             f"{XLNET_HEAD_SHAPES[name](hidden)}")
        setattr(out, name, t.data_ptr())
    return out


def xlnet_squad_head(x, weights, cls_index, start_positions, end_positions, is_impossible, p_mask, dropout_mask=None, grads=None,
                     need_dx=True, loss_scale=1.0):
    """XLnetLoss.call (xlnet/losses/xlnet_loss.py:36-120) on the last stage's content stream ``x [seq, batch, hidden]``:
    returns (loss [1] fp32 on the device, start_logits [batch, seq], end_logits [batch, seq], cls_logits [batch], dx or None).
    ``weights`` / ``grads``: dicts of fp32 tensors keyed by XLNET_HEAD_SHAPES (Dense kernels with one output as vectors);
    ``grads`` are added to in place.  ``dropout_mask [batch, hidden]`` is the factor of the dropout at :103 (None = ones)."""
    _need_cuda(x, cls_index, start_positions, end_positions, is_impossible, p_mask)
    if x.dim() != 3 or not x.is_contiguous():
        raise ValueError("xlnet_squad_head: x must be contiguous [seq, batch, hidden]")
    seq, batch, hidden = x.shape
    for t in (cls_index, start_positions, end_positions):
        if t.dtype != torch.int32 or t.numel() != batch:
            raise ValueError("xlnet_squad_head: cls_index, start_positions, end_positions must be int32 [batch]")
    for t, n in ((is_impossible, batch), (p_mask, batch * seq)) + (((dropout_mask, batch * hidden),) if dropout_mask is not None else ()):
        if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n:
            raise ValueError("xlnet_squad_head: is_impossible [batch], p_mask [batch, seq], dropout_mask [batch, hidden] must be contiguous fp32")
    wp = _xlnet_head_params(weights, hidden, "weights")
    gp = _xlnet_head_params(grads, hidden, "grads") if grads is not None else None
    lib = _lib.load()
    f32 = dict(dtype=torch.float32, device=x.device)
    nbytes = lib.ds_xlnet_squad_head_workspace_bytes(dtype_code(x), seq, batch, hidden)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    loss, sl, el, cl = torch.empty(1, **f32), torch.empty(batch, seq, **f32), torch.empty(batch, seq, **f32), torch.empty(batch, **f32)
    dx = torch.empty_like(x) if need_dx else None
    check(lib.ds_xlnet_squad_head(dtype_code(x), seq, batch, hidden, ptr(x), C.byref(wp), ptr(cls_index), ptr(start_positions),
                                  ptr(end_positions), ptr(is_impossible), ptr(p_mask), ptr(dropout_mask), loss_scale, ptr(loss), ptr(sl),
                                  ptr(el), ptr(cl), ptr(dx), C.byref(gp) if gp is not None else None, ptr(ws), nbytes,
                                  _lib.current_stream()), "ds_xlnet_squad_head")
    return loss, sl, el, cl, dx


def nmt_loss_head(x, proj_kernel, target_output, target_sequence_length, d_proj_kernel=None, need_dx=True, loss_batch_size=0,
                  loss_scale=1.0):
    """GNMT output projection + loss (gnmt/nmt/model.py:685-686, :824-838) on the last decoder cell's outputs
    ``x [seq, batch, units]`` fp32: returns (loss [1] on the device, dx or None); ``d_proj_kernel`` is added to in place."""
    _need_cuda(x, proj_kernel, target_output, target_sequence_length)
    if x.dim() != 3 or x.dtype != torch.float32 or not x.is_contiguous():
        raise ValueError("nmt_loss_head: x must be contiguous fp32 [seq, batch, units]")
    seq, batch, units = x.shape
    if proj_kernel.dtype != torch.float32 or not proj_kernel.is_contiguous() or proj_kernel.dim() != 2 or proj_kernel.shape[0] != units:
        raise ValueError("nmt_loss_head: proj_kernel must be contiguous fp32 [units, vocab]")
    vocab = proj_kernel.shape[1]
    if target_output.dtype != torch.int32 or tuple(target_output.shape) != (batch, seq) or not target_output.is_contiguous():
        raise ValueError("nmt_loss_head: target_output must be contiguous int32 [batch, seq]")
    if target_sequence_length.dtype != torch.int32 or target_sequence_length.numel() != batch:
        raise ValueError("nmt_loss_head: target_sequence_length must be int32 [batch]")
    if d_proj_kernel is not None and (d_proj_kernel.dtype != torch.float32 or not d_proj_kernel.is_contiguous()
                                      or d_proj_kernel.shape != proj_kernel.shape):
        raise ValueError("nmt_loss_head: d_proj_kernel must match proj_kernel")
    lib = _lib.load()
    nbytes = lib.ds_nmt_loss_head_workspace_bytes(seq, batch, vocab)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    loss = torch.empty(1, dtype=torch.float32, device=x.device)
    dx = torch.empty_like(x) if need_dx else None
    check(lib.ds_nmt_loss_head(seq, batch, units, vocab, ptr(x), ptr(proj_kernel), ptr(target_output), ptr(target_sequence_length),
                               loss_batch_size, loss_scale, ptr(loss), ptr(dx), ptr(d_proj_kernel), ptr(ws), nbytes,
                               _lib.current_stream()), "ds_nmt_loss_head")
    return loss, dx


VGG_HEAD_NAMES = ("fc1/kernel", "fc1/bias", "fc2/kernel", "fc2/bias", "predictions/kernel", "predictions/bias")


def vgg_head(x, weights, labels, grads=None, need_dx=True, loss_mode="as_written", loss_scale=1.0):
    """Classification block + loss of the last VGG19 stage (vgg19/applications/vgg19_slice_model.py:217-220, 342-355) on
    the flattened pool output ``x [batch, features]`` fp32.  ``weights``: {keras name: tensor} for ``VGG_HEAD_NAMES``
    (kernels ``[in, out]``); ``labels`` fp32 ``[batch]``; ``grads`` (optional, same names) are added to in place.
    ``loss_mode``: "as_written" (the reference's expression: a constant, see ds_vgg_head) or "sparse_ce".
    Returns (loss [1] on the device, probabilities [batch, classes], dx or None)."""
    w = [weights[n] for n in VGG_HEAD_NAMES]
    g = [None] * 6 if grads is None else [grads[n] for n in VGG_HEAD_NAMES]
    _need_cuda(x, labels, *w, *g)
    if x.dim() != 2 or x.dtype != torch.float32 or not x.is_contiguous():
        raise ValueError("vgg_head: x must be contiguous fp32 [batch, features]")
    batch, features = x.shape
    fc, classes = w[0].shape[1], w[4].shape[1]
    want = [(features, fc), (fc,), (fc, fc), (fc,), (fc, classes), (classes,)]
    for n, t, shp, gt in zip(VGG_HEAD_NAMES, w, want, g):
        if t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape) != shp:
            raise ValueError("vgg_head: %s must be contiguous fp32 %s" % (n, shp))
        if gt is not None and (gt.dtype != torch.float32 or not gt.is_contiguous() or gt.shape != t.shape):
            raise ValueError("vgg_head: gradient of %s must match it" % n)
    if labels.dtype != torch.float32 or labels.numel() != batch or not labels.is_contiguous():
        raise ValueError("vgg_head: labels must be contiguous fp32 [batch]")
    modes = {"as_written": _lib.DS_VGG_LOSS_AS_WRITTEN, "sparse_ce": _lib.DS_VGG_LOSS_SPARSE_CE}
    if loss_mode not in modes:
        raise ValueError("vgg_head: loss_mode %r" % (loss_mode,))
    lib = _lib.load()
    nbytes = lib.ds_vgg_head_workspace_bytes(batch, fc, classes)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    loss = torch.empty(1, dtype=torch.float32, device=x.device)
    probs = torch.empty(batch, classes, dtype=torch.float32, device=x.device)
    dx = torch.empty_like(x) if need_dx else None
    check(lib.ds_vgg_head(batch, features, fc, classes, ptr(x), *[ptr(t) for t in w], ptr(labels), modes[loss_mode], loss_scale,
                          ptr(loss), ptr(probs), ptr(dx), *[ptr(t) for t in g], ptr(ws), nbytes, _lib.current_stream()), "ds_vgg_head")
    return loss, probs, dx
