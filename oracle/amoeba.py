"""CPU restatement of one AmoebaNet cell (test infrastructure: only tests/ may import this).

Follows amoeba_net/network_utils_slice.py of the reference: ``BaseCell.__call__`` (:394-428), ``_cell_base`` (:345-378),
``_reduce_prev_layer`` (:315-343), ``_apply_operation`` (:474-521), ``_apply_conv_operation`` (:430-472),
``_stacked_separable_conv`` (:213-238), ``_pooling`` (:262-276), ``_combine_unused_states`` (:523-555) and ``batch_norm``
in training mode (:600-806), with the arg scope of model_builder_slice.py:233-290 (no biases, no activation inside the
convolutions, batch norm with scale and centre, epsilon 1e-3).  Stride 1 only (normal cells); drop path is the identity at
the driver's default ``drop_connect_keep_prob = 1.0`` (amoeba-dapple.py:128).

Tensors are NHWC torch tensors (fp64 for the checker).  The arithmetic lives in TensorFlow (slim.conv2d,
slim.separable_conv2d, tf.nn.fused_batch_norm, slim pooling), which the reference does not vendor: every function below
restates the published definition and is pinned by scalar loops on small inputs in tests/test_oracle_amoeba.py - "parity
unpinned" against TensorFlow itself.
"""
import torch
import torch.nn.functional as F

EPS = 1e-3


def relu(x):
    return torch.relu(x)


def conv1x1(x, w):
    """slim.conv2d(x, f, 1) without bias: w [cin, cout]."""
    return x @ w


def conv2d_same(x, w):
    """slim.conv2d(x, f, [kh, kw]), stride 1, 'SAME', no bias: w [kh, kw, cin, cout] (TensorFlow's layout), odd kh, kw."""
    kh, kw = w.shape[0], w.shape[1]
    y = F.conv2d(x.permute(0, 3, 1, 2), w.permute(3, 2, 0, 1), padding=(kh // 2, kw // 2))
    return y.permute(0, 2, 3, 1)


def depthwise_same(x, w):
    """The depthwise half of slim.separable_conv2d(depth_multiplier=1): w [k, k, c]."""
    k, c = w.shape[0], w.shape[2]
    y = F.conv2d(x.permute(0, 3, 1, 2), w.permute(2, 0, 1).unsqueeze(1), padding=k // 2, groups=c)
    return y.permute(0, 2, 3, 1)


def batch_norm_train(x, gamma, beta, eps=EPS):
    """tf.nn.fused_batch_norm on the batch's own moments (:765-766): biased variance over n, h, w."""
    mean = x.mean(dim=(0, 1, 2))
    var = ((x - mean) ** 2).mean(dim=(0, 1, 2))
    return (x - mean) / torch.sqrt(var + eps) * gamma + beta


def moving_average_update(moving_mean, moving_var, x, decay):
    """assign_moving_average(zero_debias=False) (:779-790); fused_batch_norm returns the unbiased variance in training."""
    n = x.shape[0] * x.shape[1] * x.shape[2]
    mean = x.mean(dim=(0, 1, 2))
    var = ((x - mean) ** 2).mean(dim=(0, 1, 2)) * (n / (n - 1) if n > 1 else 1.0)
    return moving_mean - (1 - decay) * (moving_mean - mean), moving_var - (1 - decay) * (moving_var - var)


def pool3x3(x, kind):
    """slim.avg_pool2d / max_pool2d 3 x 3, stride 1, 'SAME': the average runs over the taps inside the image."""
    xc = x.permute(0, 3, 1, 2)
    if kind == "avg":
        y = F.avg_pool2d(xc, 3, stride=1, padding=1, count_include_pad=False)
    elif kind == "max":
        y = F.max_pool2d(xc, 3, stride=1, padding=1)
    elif kind == "min":
        y = -F.max_pool2d(-xc, 3, stride=1, padding=1)
    else:
        raise NotImplementedError(kind)
    return y.permute(0, 2, 3, 1)


def _bn(x, p, scope):
    return batch_norm_train(x, p[scope + "/gamma"], p[scope + "/beta"])


def stacked_separable_conv(x, p, scope, k, num_layers):
    """:213-238: num_layers x (relu, depthwise k x k, pointwise, batch norm)."""
    for j in range(1, num_layers + 1):
        s = "%s/separable_%dx%d_%d" % (scope, k, k, j)
        x = relu(x)
        x = conv1x1(depthwise_same(x, p[s + "/depthwise_weights"]), p[s + "/pointwise_weights"])
        x = _bn(x, p, "%s/bn_sep_%dx%d_%d" % (scope, k, k, j))
    return x


def apply_operation(x, op, p, scope, filter_size):
    """:474-521 at stride 1, drop path off."""
    cin = x.shape[-1]
    if "separable" in op:
        parts = op.split("_")
        k = int(parts[1].split("x")[0])
        return stacked_separable_conv(x, p, scope, k, int(parts[2]))
    if op in ("1x7_7x1", "1x3_3x1"):
        k = int(op[2])
        reduced = int(3 * filter_size / 8) if op == "1x3_3x1" else int(filter_size / 4)
        a, b = "1x%d" % k, "%dx1" % k

        def factorised(t, width):
            t = conv2d_same(t, p["%s/%s/weights" % (scope, a)].reshape(1, k, -1, width))
            t = relu(_bn(t, p, "%s/bn_%s" % (scope, op)))
            return conv2d_same(t, p["%s/%s/weights" % (scope, b)].reshape(k, 1, width, width))
        if reduced < 1:
            return _bn(factorised(relu(x), filter_size), p, scope + "/bn")
        t = _bn(conv1x1(relu(x), p[scope + "/pre_1x1/weights"]), p, scope + "/pre_bn")
        t = _bn(factorised(relu(t), reduced), p, scope + "/bn")
        return _bn(conv1x1(relu(t), p[scope + "/post_1x1/weights"]), p, scope + "/post_bn")
    if op in ("none", "1x1"):
        if op == "1x1" or cin != filter_size:
            return _bn(conv1x1(relu(x), p[scope + "/1x1/weights"]), p, scope + "/bn_1")
        return x
    if "pool" in op:
        y = pool3x3(x, op.split("_")[0])
        if cin != filter_size:
            y = _bn(conv1x1(y, p[scope + "/1x1/weights"]), p, scope + "/bn_1")
        return y
    raise NotImplementedError(op)


def cell_head(net, prev_layer, p, scope, filter_size):
    """Up to the pipeline cut (:332-343, :353-365): the two tensors that leave the first device of a cut cell - prev_layer
    after relu + 1 x 1 (when its channel count differs, else prev_layer itself) and net after relu + 1 x 1."""
    if prev_layer is None:            # :318-319: the current layer stands in, untouched
        cut_prev = net
    elif prev_layer.shape[-1] != filter_size:
        cut_prev = conv1x1(relu(prev_layer), p[scope + "/prev_1x1/weights"])
    else:
        cut_prev = prev_layer
    cut_net = conv1x1(relu(net), p[scope + "/1x1/weights"])
    return cut_prev, cut_net


def cell_tail(cut_prev, cut_net, prev_reduced, p, scope, filter_size, operations, hiddenstate_indices, used_hiddenstates):
    """From the cut on: the two batch norms (:343, :367), the five combinations (:405-421) and the concatenation of the
    unused states (:523-555).  prev_reduced: whether cut_prev went through prev_1x1 (and therefore gets prev_bn)."""
    prev = _bn(cut_prev, p, scope + "/prev_bn") if prev_reduced else cut_prev
    states = [_bn(cut_net, p, scope + "/beginning_bn"), prev]
    for it in range(5):
        li, ri = hiddenstate_indices[2 * it], hiddenstate_indices[2 * it + 1]
        h1 = apply_operation(states[li], operations[2 * it], p, "%s/comb_iter_%d/left" % (scope, it), filter_size)
        h2 = apply_operation(states[ri], operations[2 * it + 1], p, "%s/comb_iter_%d/right" % (scope, it), filter_size)
        states.append(h1 + h2)
    final = states[-1].shape[-1]
    for idx, used in enumerate(used_hiddenstates):   # :531-547: an unused state of another width is brought to the final one
        if not used and states[idx].shape[-1] != final:
            s_ = "%s/cell_output/reduction_%d" % (scope, idx)
            states[idx] = _bn(conv1x1(states[idx], p[s_ + "/path_conv/weights"]), p, s_ + "/path_bn")
    return torch.cat([h for h, used in zip(states, used_hiddenstates) if not used], dim=-1)


def cell_forward(net, prev_layer, p, scope, filter_size, operations, hiddenstate_indices, used_hiddenstates):
    """BaseCell.__call__ at stride 1 -> (output, (cut_prev, cut_net))."""
    reduced = prev_layer is not None and prev_layer.shape[-1] != filter_size
    cut_prev, cut_net = cell_head(net, prev_layer, p, scope, filter_size)
    out = cell_tail(cut_prev, cut_net, reduced, p, scope, filter_size, operations, hiddenstate_indices, used_hiddenstates)
    return out, (cut_prev, cut_net)


def cell_vjp(net, prev_layer, p, d_out, scope, filter_size, operations, hiddenstate_indices, used_hiddenstates):
    """Output, input gradients (d_net, d_prev) and parameter gradients of the cell for the upstream gradient d_out."""
    net = net.clone().requires_grad_(True)
    prev = None if prev_layer is None else prev_layer.clone().requires_grad_(True)
    names = sorted(n for n in p if n.startswith(scope + "/") and "moving_" not in n)
    params = {n: p[n].clone().requires_grad_(True) for n in names}
    full = dict(p)
    full.update(params)
    out, _ = cell_forward(net, prev, full, scope, filter_size, operations, hiddenstate_indices, used_hiddenstates)
    ins = [net] + ([prev] if prev is not None else []) + [params[n] for n in names]
    grads = torch.autograd.grad(out, ins, d_out, allow_unused=True)
    d_net = grads[0]
    d_prev = grads[1] if prev is not None else None
    off = 2 if prev is not None else 1
    dw = {n: (g if g is not None else torch.zeros_like(params[n])) for n, g in zip(names, grads[off:])}
    return out.detach(), d_net, d_prev, dw
