"""Optimizers of the reference over a stage's flat fp32 master buffers (one fused HIP launch per step).

Same class names and keyword arguments as the reference: ``AdamWeightDecayOptimizer``
(bert/graph_helper.py:191-272), ``AdamOptimizer`` / ``GradientDescentOptimizer`` (tf.train, as used by
xlnet/utils/xlnet_utils.py:195-197 and vgg19/tf-keras-dapple.py:187).  ``apply_gradients`` takes the stage
whose ``grads`` hold the accumulated gradients - or a list of parameter sets (the stages of a pipeline plus
``FlatParams`` for head weights kept outside a stage): ``max_gradient_norm`` is the flag of bert/graph.py:162-165,
``tf.clip_by_global_norm`` over the gradients of ALL slices, so with a list the norm is taken over every set and
the same factor scales each of them.  After a step a stage's compute copies are stale; ``apply_gradients`` marks
the stage and its next forward pass rebuilds them (``Stage.refresh_weights``).
"""
import ctypes as C
import re

import torch

from . import _lib
from ._lib import check


class FlatParams:
    """Named fp32 tensors packed like a stage's master buffers (every tensor 256-byte aligned), for parameters
    that live outside a stage handle.  Offers the attributes the optimizers read from a ``runtime.Stage``."""

    def __init__(self, named, device="cuda:0"):
        self.device = torch.device(device)
        self.weight_names = list(named)
        self.weight_numels = [int(torch.as_tensor(named[n]).numel()) for n in self.weight_names]
        sizes = [(k + 63) // 64 * 64 for k in self.weight_numels]
        self.weight_offsets = [sum(sizes[:i]) for i in range(len(sizes))]
        self.flat_weights = torch.zeros(sum(sizes), dtype=torch.float32, device=self.device)
        self.flat_grads = torch.zeros_like(self.flat_weights)
        self.weights, self.grads = {}, {}
        for n, off, k in zip(self.weight_names, self.weight_offsets, self.weight_numels):
            t = torch.as_tensor(named[n], dtype=torch.float32)
            self.weights[n] = self.flat_weights[off:off + k].view(t.shape)
            self.weights[n].copy_(t)
            self.grads[n] = self.flat_grads[off:off + k].view(t.shape)


class _FlatOptimizer:
    def __init__(self):
        self.lib = _lib.load()
        self._plans = {}        # id(stage) -> (plan handle, state tensors)
        self._sq = None

    def _decay_rate(self, name):
        return 0.0

    def _plan(self, stage):
        key = id(stage)
        if key not in self._plans:
            n = len(stage.weight_names)
            offs = (C.c_int64 * n)(*stage.weight_offsets)
            nums = (C.c_int64 * n)(*stage.weight_numels)
            dec = (C.c_float * n)(*[self._decay_rate(nm) for nm in stage.weight_names])
            h = C.c_void_p()
            check(self.lib.ds_optim_plan_create(n, offs, nums, dec, C.byref(h)), "ds_optim_plan_create")
            self._plans[key] = (h, self._new_state(stage))
        return self._plans[key]

    def _new_state(self, stage):
        return ()

    def global_sqnorm(self, sets):
        """Device scalar (fp64) holding sum(g^2) over the gradients of every parameter set in ``sets``: the square of
        the global norm tf.clip_by_global_norm takes over grads_set (bert/graph.py:162-165)."""
        sets = list(sets)
        if self._sq is None:
            self._sq = torch.zeros(1, dtype=torch.float64, device=sets[0].device)
        self._sq.zero_()
        for st in sets:
            check(self.lib.ds_grad_sqnorm_accum(_lib.ptr(st.flat_grads), st.flat_grads.numel(), _lib.ptr(self._sq),
                                                _lib.current_stream()), "ds_grad_sqnorm_accum")
        return self._sq

    def apply_gradients(self, params, max_gradient_norm=None, learning_rate=None):
        """``params``: a ``runtime.Stage`` / ``FlatParams``, or a list of them clipped by their common global norm."""
        sets = list(params) if isinstance(params, (list, tuple)) else [params]
        sq = None if max_gradient_norm is None else self.global_sqnorm(sets)
        for st in sets:
            self._apply(st, sq, max_gradient_norm, learning_rate)
            if hasattr(st, "mark_weights_stale"):
                st.mark_weights_stale()

    def close(self):
        for h, _ in self._plans.values():
            self.lib.ds_optim_plan_destroy(h)
        self._plans = {}

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class AdamWeightDecayOptimizer(_FlatOptimizer):
    """bert/graph_helper.py:194-211 constructor arguments; :213-272 update."""

    def __init__(self, learning_rate, weight_decay_rate=0.0, beta_1=0.9, beta_2=0.999, epsilon=1e-6,
                 exclude_from_weight_decay=None, name="AdamWeightDecayOptimizer"):
        super().__init__()
        self.learning_rate = learning_rate
        self.weight_decay_rate = weight_decay_rate
        self.beta_1, self.beta_2, self.epsilon = beta_1, beta_2, epsilon
        self.exclude_from_weight_decay = exclude_from_weight_decay
        self.name = name

    def _do_use_weight_decay(self, param_name):
        """bert/graph_helper.py:274-282."""
        if not self.weight_decay_rate:
            return False
        if self.exclude_from_weight_decay:
            for r in self.exclude_from_weight_decay:
                if re.search(r, param_name) is not None:
                    return False
        return True

    def _decay_rate(self, name):
        return float(self.weight_decay_rate) if self._do_use_weight_decay(name) else 0.0

    def _new_state(self, stage):
        return (torch.zeros_like(stage.flat_weights), torch.zeros_like(stage.flat_weights))   # adam_m, adam_v (:223-234)

    def _apply(self, stage, sq, max_gradient_norm, learning_rate):
        plan, (m, v) = self._plan(stage)
        lr = self.learning_rate if learning_rate is None else learning_rate
        check(self.lib.ds_adam_step(plan, _lib.ptr(stage.flat_weights), _lib.ptr(stage.flat_grads), _lib.ptr(m), _lib.ptr(v),
                                    lr, self.beta_1, self.beta_2, self.epsilon, _lib.ptr(sq),
                                    0.0 if max_gradient_norm is None else max_gradient_norm, _lib.current_stream()), "ds_adam_step")

    def moments(self, stage):
        return self._plan(stage)[1]


class AdamOptimizer(_FlatOptimizer):
    """tf.train.AdamOptimizer(learning_rate, beta1, beta2, epsilon) of xlnet/utils/xlnet_utils.py:195-197."""

    def __init__(self, learning_rate=0.001, beta1=0.9, beta2=0.999, epsilon=1e-8, name="Adam"):
        super().__init__()
        self.learning_rate, self.beta1, self.beta2, self.epsilon, self.name = learning_rate, beta1, beta2, epsilon, name
        self._t = {}

    def _new_state(self, stage):
        return (torch.zeros_like(stage.flat_weights), torch.zeros_like(stage.flat_weights))

    def _apply(self, stage, sq, max_gradient_norm, learning_rate):
        plan, (m, v) = self._plan(stage)
        t = self._t[id(stage)] = self._t.get(id(stage), 0) + 1
        lr = self.learning_rate if learning_rate is None else learning_rate
        lr_t = lr * (1.0 - self.beta2 ** t) ** 0.5 / (1.0 - self.beta1 ** t)
        check(self.lib.ds_adam_step(plan, _lib.ptr(stage.flat_weights), _lib.ptr(stage.flat_grads), _lib.ptr(m), _lib.ptr(v),
                                    lr_t, self.beta1, self.beta2, self.epsilon, _lib.ptr(sq),
                                    0.0 if max_gradient_norm is None else max_gradient_norm, _lib.current_stream()), "ds_adam_step")


class GradientDescentOptimizer(_FlatOptimizer):
    """tf.train.GradientDescentOptimizer(learning_rate) of vgg19/tf-keras-dapple.py:187."""

    def __init__(self, learning_rate, name="GradientDescent"):
        super().__init__()
        self.learning_rate, self.name = learning_rate, name

    def _apply(self, stage, sq, max_gradient_norm, learning_rate):
        plan, _ = self._plan(stage)
        lr = self.learning_rate if learning_rate is None else learning_rate
        check(self.lib.ds_sgd_step(plan, _lib.ptr(stage.flat_weights), _lib.ptr(stage.flat_grads), lr, _lib.ptr(sq),
                                   0.0 if max_gradient_norm is None else max_gradient_norm, _lib.current_stream()), "ds_sgd_step")


def xlnet_learning_rate(global_step, learning_rate, warmup_steps, train_steps, min_lr_ratio):
    """Host-side schedule of xlnet/utils/xlnet_utils.py:179-193 (linear warm-up below step 1000, then linear decay)."""
    warmup_lr = float(global_step) / float(warmup_steps) * learning_rate
    end = learning_rate * min_lr_ratio
    decay_steps = train_steps - warmup_steps
    if decay_steps <= 0:
        decay_lr = end
    else:
        s = min(max(global_step - warmup_steps, 0), decay_steps)
        decay_lr = (learning_rate - end) * (1.0 - float(s) / decay_steps) + end
    return warmup_lr if global_step < 1000 else decay_lr
