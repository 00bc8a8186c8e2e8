"""One AmoebaNet cell on the GPU: ``BaseCell.__call__`` of amoeba_net/network_utils_slice.py:394-428 composed from the
library's operators (``ds_relu_*``, ``ds_batchnorm_train_*``, ``ds_pool3x3_*``, ``ds_depthwise_conv_*``, ``ds_gather1d`` /
``ds_scatter1d``, ``ds_add``, ``ds_copy2d`` and ``ds_gemm`` for every 1 x 1, pointwise and gathered convolution), with the
backward pass over the same graph in reverse.  fp32, NHWC, stride 1 (normal cells); drop path at the driver's default keep
probability 1.0 (amoeba-dapple.py:128) is the identity.  torch only owns the buffers.

Parameters live in a dict under the reference's variable names without the ``:0`` (``cell_3/1x1/weights``,
``cell_3/comb_iter_0/left/separable_3x3_1/depthwise_weights`` ...): 1 x 1 and pointwise kernels as ``[cin, cout]``, depthwise
kernels as ``[k, k, c]``, the 1 x k and k x 1 kernels as ``[k * cin, cout]`` (TensorFlow's ``[1, k, cin, cout]`` /
``[k, 1, cin, cout]`` read row-major), batch norm ``gamma`` / ``beta`` / ``moving_mean`` / ``moving_variance`` as ``[c]``.
Gradients are ADDED to a dict of the same names (the accumulation over micro-batches of amoeba_net_slice_model.py:393-462).
"""
import ctypes as C

import torch

from . import _lib
from ._lib import DS_K_MAJOR, DS_MN_MAJOR, DS_EPI_ACCUM, check, ptr
from . import ops

BN_EPSILON = 1e-3       # model_builder_slice.py:235
BN_DECAY = 0.9997       # model_builder_slice.py:234


def _f32(t, what):
    if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous():
        raise ValueError("%s must be a contiguous fp32 tensor on the GPU" % what)
    return t


def operation_shapes(op, cin, filter_size):
    """[(variable suffix, shape)] of one operation of a cell at stride 1 (``_apply_operation``, :474-521)."""
    out = []

    def bn(name, c):
        out.extend([(name + "/gamma", (c,)), (name + "/beta", (c,)), (name + "/moving_mean", (c,)), (name + "/moving_variance", (c,))])
    if "separable" in op:
        parts = op.split("_")
        k, layers = int(parts[1].split("x")[0]), int(parts[2])
        c = cin
        for j in range(1, layers + 1):
            out.append(("separable_%dx%d_%d/depthwise_weights" % (k, k, j), (k, k, c)))
            out.append(("separable_%dx%d_%d/pointwise_weights" % (k, k, j), (c, filter_size)))
            bn("bn_sep_%dx%d_%d" % (k, k, j), filter_size)
            c = filter_size
    elif op in ("1x7_7x1", "1x3_3x1"):
        k = int(op[2])
        reduced = int(3 * filter_size / 8) if op == "1x3_3x1" else int(filter_size / 4)
        width, c = (reduced, reduced) if reduced >= 1 else (filter_size, cin)
        if reduced >= 1:
            out.append(("pre_1x1/weights", (cin, reduced)))
            bn("pre_bn", reduced)
        out.append(("1x%d/weights" % k, (k * c, width)))
        bn("bn_" + op, width)
        out.append(("%dx1/weights" % k, (k * width, width)))
        bn("bn", width)
        if reduced >= 1:
            out.append(("post_1x1/weights", (reduced, filter_size)))
            bn("post_bn", filter_size)
    elif op in ("none", "1x1"):
        if op == "1x1" or cin != filter_size:
            out.append(("1x1/weights", (cin, filter_size)))
            bn("bn_1", filter_size)
    elif "pool" in op:
        if cin != filter_size:
            out.append(("1x1/weights", (cin, filter_size)))
            bn("bn_1", filter_size)
    else:
        raise NotImplementedError("operation %r is not built" % op)
    return out


def cell_variable_shapes(scope, net_channels, prev_channels, filter_size, operations, hiddenstate_indices, used_hiddenstates):
    """{variable name: shape} of a cell called with ``net`` of net_channels and ``prev_layer`` of prev_channels (None: no
    prev_layer) - what ``slim`` would create under the cell's variable scope."""
    shapes = {}

    def bn(name, c):
        for s in ("gamma", "beta", "moving_mean", "moving_variance"):
            shapes["%s/%s/%s" % (scope, name, s)] = (c,)
    widths = [filter_size, net_channels if prev_channels is None else filter_size]
    if prev_channels is not None and prev_channels != filter_size:
        shapes[scope + "/prev_1x1/weights"] = (prev_channels, filter_size)
        bn("prev_bn", filter_size)
    shapes[scope + "/1x1/weights"] = (net_channels, filter_size)
    bn("beginning_bn", filter_size)
    for it in range(5):
        for side, j in (("left", 2 * it), ("right", 2 * it + 1)):
            for name, shp in operation_shapes(operations[j], widths[hiddenstate_indices[j]], filter_size):
                shapes["%s/comb_iter_%d/%s/%s" % (scope, it, side, name)] = shp
        widths.append(filter_size)
    for idx, used in enumerate(used_hiddenstates):
        if not used and widths[idx] != filter_size:
            shapes["%s/cell_output/reduction_%d/path_conv/weights" % (scope, idx)] = (widths[idx], filter_size)
            bn("cell_output/reduction_%d/path_bn" % idx, filter_size)
    return shapes


class _Graph:
    """The operations of one forward pass in order, each with the closure that runs its backward step."""

    def __init__(self, params, grads, is_training=True):
        self.p, self.g = params, grads
        self.lib = _lib.load()
        self.stream = _lib.current_stream()
        self.tape = []
        self.grad = {}          # id(tensor) -> gradient buffer
        self.keep = []          # tensors the closures refer to by id
        self.is_training = is_training

    # ---- gradient bookkeeping: the first contribution writes, later ones add
    def _into(self, x, launch):
        key = id(x)
        if key in self.grad:
            launch(self.grad[key], 1)
        else:
            buf = torch.empty_like(x)
            self.grad[key] = buf
            launch(buf, 0)

    def _take(self, y):
        """The gradient that has arrived at y (None: nothing downstream depends on it)."""
        return self.grad.pop(id(y), None)

    def _param(self, name):
        return _f32(self.p[name], name)

    def _pgrad(self, name):
        return _f32(self.g[name], "gradient of " + name) if self.g is not None and name in self.g else None

    def _new(self, *shape):
        return torch.empty(*shape, dtype=torch.float32, device="cuda")

    def _gemm(self, a, b, c, m, n, k, am, bm, accumulate=False):
        ops.gemm(a, b, c, m, n, k, am, bm, flags=DS_EPI_ACCUM if accumulate else 0)

    # ---- operators
    def relu(self, x):
        y = torch.empty_like(x)
        check(self.lib.ds_relu_fwd(x.numel(), ptr(x), ptr(y), self.stream), "ds_relu_fwd")

        def bwd():
            dy = self._take(y)
            if dy is None:
                return
            self._into(x, lambda dx, acc: check(self.lib.ds_relu_bwd(x.numel(), ptr(x), ptr(dy), ptr(dx), acc, self.stream), "ds_relu_bwd"))
        self.tape.append(bwd)
        self.keep.append(y)
        return y

    def matmul(self, x2d, wname):
        """x2d [rows, cin] x weights [cin, cout]: a 1 x 1 / pointwise / gathered convolution as ds_gemm."""
        w = self._param(wname)
        rows, cin = x2d.shape
        cout = w.shape[1]
        if w.shape[0] != cin or cin % 4 or cout % 4:
            raise ValueError("%s: kernel %s does not fit %d input channels (channel counts must be multiples of 4)" % (wname, tuple(w.shape), cin))
        y = self._new(rows, cout)
        self._gemm(x2d, w, y, rows, cout, cin, DS_K_MAJOR, DS_MN_MAJOR)

        def bwd():
            dy = self._take(y)
            if dy is None:
                return
            dw = self._pgrad(wname)
            if dw is not None:      # dw[cin, cout] += x^T dy
                self._gemm(x2d, dy, dw, cin, cout, rows, DS_MN_MAJOR, DS_MN_MAJOR, accumulate=True)
            # dx[rows, cin] (+)= dy w^T
            self._into(x2d, lambda dx, acc: self._gemm(dy, w, dx, rows, cin, cout, DS_K_MAJOR, DS_K_MAJOR, accumulate=bool(acc)))
        self.tape.append(bwd)
        self.keep.append(y)
        return y

    def conv1x1(self, x, wname):
        n, h, w_, c = x.shape
        x2 = x.view(n * h * w_, c)
        self._alias(x, x2)
        y2 = self.matmul(x2, wname)
        y = y2.view(n, h, w_, -1)
        self._alias(y2, y)
        return y

    def _alias(self, a, b):
        """b is a view of a: both names share one gradient buffer (viewed the same way)."""
        self.keep.extend([a, b])

        def bwd():
            if id(b) in self.grad:
                gb = self.grad.pop(id(b))
                ga = gb.view(a.shape)
                if id(a) in self.grad:
                    dst = self.grad[id(a)]
                    check(self.lib.ds_copy2d(1, a.numel(), ptr(ga), a.numel(), ptr(dst), a.numel(), 1, self.stream), "ds_copy2d")
                else:
                    self.grad[id(a)] = ga
        self.tape.append(bwd)

    def conv1d(self, x, wname, k, axis):
        """slim.conv2d(x, f, [1, k]) (axis 1) / [k, 1] (axis 0), stride 1, 'SAME', as a gather and a GEMM."""
        n, h, w_, c = x.shape
        col = self._new(n * h * w_, k * c)
        check(self.lib.ds_gather1d(n, h, w_, c, k, axis, ptr(x), ptr(col), self.stream), "ds_gather1d")
        y2 = self.matmul(col, wname)

        def bwd():
            if id(col) not in self.grad:
                return
            dcol = self.grad.pop(id(col))
            self._into(x, lambda dx, acc: check(self.lib.ds_scatter1d(n, h, w_, c, k, axis, ptr(dcol), ptr(dx), acc, self.stream), "ds_scatter1d"))
        # (the tape runs backwards: this closure, pushed before matmul's, would run after it - so it is inserted beneath)
        self.tape.insert(len(self.tape) - 1, bwd)
        y = y2.view(n, h, w_, -1)
        self._alias(y2, y)
        return y

    def depthwise(self, x, wname):
        w = self._param(wname)
        n, h, w_, c = x.shape
        k = w.shape[0]
        if tuple(w.shape) != (k, k, c):
            raise ValueError("%s: depthwise kernel %s does not fit %d channels" % (wname, tuple(w.shape), c))
        y = torch.empty_like(x)
        check(self.lib.ds_depthwise_conv_fwd(n, h, w_, c, k, ptr(x), ptr(w), ptr(y), self.stream), "ds_depthwise_conv_fwd")

        def bwd():
            dy = self._take(y)
            if dy is None:
                return
            dw = self._pgrad(wname)
            self._into(x, lambda dx, acc: check(self.lib.ds_depthwise_conv_bwd(n, h, w_, c, k, ptr(x), ptr(w), ptr(dy), ptr(dx), acc, ptr(dw),
                                                                               self.stream), "ds_depthwise_conv_bwd"))
        self.tape.append(bwd)
        self.keep.append(y)
        return y

    def batch_norm(self, x, scope):
        gamma, beta = self._param(scope + "/gamma"), self._param(scope + "/beta")
        c = x.shape[-1]
        rows = x.numel() // c
        y = torch.empty_like(x)
        mean, rstd = self._new(c), self._new(c)
        ws = torch.empty(self.lib.ds_batchnorm_workspace_bytes(c), dtype=torch.uint8, device="cuda")
        mm = self.p.get(scope + "/moving_mean") if self.is_training else None
        mv = self.p.get(scope + "/moving_variance") if self.is_training else None
        check(self.lib.ds_batchnorm_train_fwd(rows, c, ptr(x), ptr(gamma), ptr(beta), BN_EPSILON, ptr(y), ptr(mean), ptr(rstd), ptr(mm), ptr(mv),
                                              BN_DECAY, ptr(ws), self.stream), "ds_batchnorm_train_fwd")

        def bwd():
            dy = self._take(y)
            if dy is None:
                return
            dg, db = self._pgrad(scope + "/gamma"), self._pgrad(scope + "/beta")
            self._into(x, lambda dx, acc: check(self.lib.ds_batchnorm_train_bwd(rows, c, ptr(dy), ptr(x), ptr(gamma), ptr(mean), ptr(rstd), ptr(dx), acc,
                                                                                ptr(dg), ptr(db), ptr(ws), self.stream), "ds_batchnorm_train_bwd"))
        self.tape.append(bwd)
        self.keep.extend([y, ws])
        return y

    def pool(self, x, kind):
        n, h, w_, c = x.shape
        if kind not in ("avg", "max"):
            raise NotImplementedError("%s pooling is not used by the cell specifications of model_specs.py and is not built" % kind)
        src = x
        code = 0 if kind == "avg" else 1
        y = torch.empty_like(src)
        check(self.lib.ds_pool3x3_fwd(code, n, h, w_, c, ptr(src), ptr(y), self.stream), "ds_pool3x3_fwd")

        def bwd():
            dy = self._take(y)
            if dy is None:
                return
            self._into(src, lambda dx, acc: check(self.lib.ds_pool3x3_bwd(code, n, h, w_, c, ptr(src), ptr(dy), ptr(dx), acc, self.stream), "ds_pool3x3_bwd"))
        self.tape.append(bwd)
        self.keep.append(y)
        return y

    def add(self, a, b):
        y = torch.empty_like(a)
        check(self.lib.ds_add(a.numel(), ptr(a), ptr(b), ptr(y), self.stream), "ds_add")

        def bwd():
            dy = self._take(y)
            if dy is None:
                return
            for t in (a, b):
                self._into(t, lambda d, acc: check(self.lib.ds_copy2d(1, t.numel(), ptr(dy), t.numel(), ptr(d), t.numel(), acc, self.stream), "ds_copy2d"))
        self.tape.append(bwd)
        self.keep.append(y)
        return y

    def concat(self, parts):
        n, h, w_, _ = parts[0].shape
        rows = n * h * w_
        total = sum(t.shape[-1] for t in parts)
        y = self._new(n, h, w_, total)
        offs, o = [], 0
        for t in parts:
            c = t.shape[-1]
            check(self.lib.ds_copy2d(rows, c, ptr(t), c, y.data_ptr() + 4 * o, total, 0, self.stream), "ds_copy2d")
            offs.append(o)
            o += c

        def bwd():
            dy = self._take(y)
            if dy is None:
                return
            for t, o_ in zip(parts, offs):
                c = t.shape[-1]
                self._into(t, lambda d, acc: check(self.lib.ds_copy2d(rows, c, dy.data_ptr() + 4 * o_, total, ptr(d), c, acc, self.stream), "ds_copy2d"))
        self.tape.append(bwd)
        self.keep.append(y)
        return y

    def backward(self, out, d_out, wanted):
        """Runs the tape in reverse from d out; returns the gradients of the tensors in `wanted` (None where none flowed)."""
        self.grad[id(out)] = _f32(d_out, "d_out").clone()
        for step in reversed(self.tape):
            step()
        return [self.grad.get(id(t)) for t in wanted]


class Cell:
    """The cell of ``BaseCell.__call__`` for one call: ``forward`` and ``backward`` on NHWC fp32 tensors."""

    def __init__(self, scope, filter_size, operations, hiddenstate_indices, used_hiddenstates, params, grads=None):
        self.scope, self.f = scope, int(filter_size)
        self.ops, self.idx, self.used = list(operations), list(hiddenstate_indices), list(used_hiddenstates)
        if len(self.ops) != 10 or len(self.idx) != 10 or len(self.used) != 7:
            raise ValueError("a cell has 10 operations, 10 hidden-state indices and 7 used flags")
        self.params, self.grads = params, grads
        self.cut_outputs = None
        self._graph = None

    def _apply(self, g, x, op, scope):
        """``_apply_operation`` (:474-521) at stride 1 with drop path off."""
        cin = x.shape[-1]
        if "separable" in op:
            parts = op.split("_")
            if op.startswith("dil"):
                raise NotImplementedError("dilated separable convolutions are not built")
            k, layers = int(parts[1].split("x")[0]), int(parts[2])
            for j in range(1, layers + 1):
                s = "%s/separable_%dx%d_%d" % (scope, k, k, j)
                x = g.conv1x1(g.depthwise(g.relu(x), s + "/depthwise_weights"), s + "/pointwise_weights")
                x = g.batch_norm(x, "%s/bn_sep_%dx%d_%d" % (scope, k, k, j))
            return x
        if op in ("1x7_7x1", "1x3_3x1"):
            k = int(op[2])
            reduced = int(3 * self.f / 8) if op == "1x3_3x1" else int(self.f / 4)

            def factorised(t):
                t = g.conv1d(t, "%s/1x%d/weights" % (scope, k), k, 1)
                t = g.relu(g.batch_norm(t, "%s/bn_%s" % (scope, op)))
                return g.conv1d(t, "%s/%dx1/weights" % (scope, k), k, 0)
            if reduced < 1:
                return g.batch_norm(factorised(g.relu(x)), scope + "/bn")
            t = g.batch_norm(g.conv1x1(g.relu(x), scope + "/pre_1x1/weights"), scope + "/pre_bn")
            t = g.batch_norm(factorised(g.relu(t)), scope + "/bn")
            return g.batch_norm(g.conv1x1(g.relu(t), scope + "/post_1x1/weights"), scope + "/post_bn")
        if op in ("none", "1x1"):
            if op == "1x1" or cin != self.f:
                return g.batch_norm(g.conv1x1(g.relu(x), scope + "/1x1/weights"), scope + "/bn_1")
            return x
        if "pool" in op:
            y = g.pool(x, op.split("_")[0])
            if cin != self.f:
                y = g.batch_norm(g.conv1x1(y, scope + "/1x1/weights"), scope + "/bn_1")
            return y
        raise NotImplementedError("operation %r is not built" % op)

    def forward(self, net, prev_layer=None, is_training=True):
        """-> the cell's output [n, h, w, f * (number of unused states)]; ``cut_outputs`` = the two tensors at the pipeline
        cut (:335, :365): prev_layer after relu + prev_1x1 (or as it came) and net after relu + 1x1."""
        _f32(net, "net")
        if prev_layer is not None:
            _f32(prev_layer, "prev_layer")
            if prev_layer.shape[1:3] != net.shape[1:3]:
                raise NotImplementedError("a prev_layer of another spatial size needs factorized_reduction (reduction cells), which is not built")
        g = _Graph(self.params, self.grads, is_training)
        s = self.scope
        reduced = prev_layer is not None and prev_layer.shape[-1] != self.f
        if prev_layer is None:
            cut_prev = net
        elif reduced:
            cut_prev = g.conv1x1(g.relu(prev_layer), s + "/prev_1x1/weights")
        else:
            cut_prev = prev_layer
        cut_net = g.conv1x1(g.relu(net), s + "/1x1/weights")
        self.cut_outputs = [cut_prev, cut_net]
        prev = g.batch_norm(cut_prev, s + "/prev_bn") if reduced else cut_prev
        states = [g.batch_norm(cut_net, s + "/beginning_bn"), prev]
        for it in range(5):
            li, ri = self.idx[2 * it], self.idx[2 * it + 1]
            h1 = self._apply(g, states[li], self.ops[2 * it], "%s/comb_iter_%d/left" % (s, it))
            h2 = self._apply(g, states[ri], self.ops[2 * it + 1], "%s/comb_iter_%d/right" % (s, it))
            states.append(g.add(h1, h2))
        for i, used in enumerate(self.used):
            if not used and states[i].shape[-1] != self.f:
                r = "%s/cell_output/reduction_%d" % (s, i)
                states[i] = g.batch_norm(g.conv1x1(states[i], r + "/path_conv/weights"), r + "/path_bn")
        out = g.concat([h for h, used in zip(states, self.used) if not used])
        self._graph, self._io = g, (out, net, prev_layer)
        return out

    def backward(self, d_out):
        """-> (d_net, d_prev_layer or None); parameter gradients are added to ``grads``."""
        if self._graph is None:
            raise RuntimeError("backward without a forward pass")
        out, net, prev = self._io
        wanted = [net] + ([prev] if prev is not None else [])
        res = self._graph.backward(out, d_out, wanted)
        self._graph = None
        zero = lambda t: torch.zeros_like(t)
        d_net = res[0] if res[0] is not None else zero(net)
        d_prev = None if prev is None else (res[1] if res[1] is not None else zero(prev))
        return d_net, d_prev
