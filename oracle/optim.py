"""CPU restatement of what the reference applies to the accumulated gradients. TEST INFRASTRUCTURE ONLY.

* clip_by_global_norm: bert/graph.py:162-165 calls tf.clip_by_global_norm(grads, clip_norm); TensorFlow
  (un-vendored, >= 1.12 < 2.0) defines it as  global_norm = sqrt(sum_t sum(t**2)),
  t_clipped = t * clip_norm / max(global_norm, clip_norm).
* AdamWeightDecayOptimizer.apply_gradients: bert/graph_helper.py:213-272 (line numbers cited per step).
* tf.train.AdamOptimizer as used by xlnet/utils/xlnet_utils.py:195-197; TensorFlow's published update:
  lr_t = lr * sqrt(1 - b2**t) / (1 - b1**t);  m, v as below;  w -= lr_t * m / (sqrt(v) + eps).
* tf.train.GradientDescentOptimizer (vgg19/tf-keras-dapple.py:187): w -= lr * g.
* the learning-rate schedule of xlnet/utils/xlnet_utils.py:179-193.

Pins (tests/test_oracle_optim.py): the reference's own known-answer test
bert/models/bert/optimization_test.py:25-44 (100 steps at lr 0.2 reach the target within 1e-2), the
hand-computed first step from zero moments, torch.optim.Adam with a vanishing epsilon for the
bias-corrected form, and brute-force clipping.  Parity unpinned by the reference: TensorFlow's Adam
epsilon placement ("epsilon hat") and polynomial_decay are restated from TensorFlow's documentation.
"""
import re

import numpy as np


def global_norm(grads):
    return float(np.sqrt(sum(float(np.sum(np.square(np.asarray(g, np.float64)))) for g in grads)))


def clip_by_global_norm(grads, clip_norm):
    """bert/graph.py:162-165."""
    norm = global_norm(grads)
    scale = clip_norm / max(norm, clip_norm)
    return [np.asarray(g) * scale for g in grads], norm


def use_weight_decay(param_name, weight_decay_rate, exclude_from_weight_decay):
    """bert/graph_helper.py:274-282."""
    if not weight_decay_rate:
        return False
    if exclude_from_weight_decay:
        for r in exclude_from_weight_decay:
            if re.search(r, param_name) is not None:
                return False
    return True


class AdamWeightDecay:
    """bert/graph_helper.py:191-272; defaults of :194-200, BERT's construction at :179-185."""

    def __init__(self, learning_rate, weight_decay_rate=0.0, beta_1=0.9, beta_2=0.999, epsilon=1e-6,
                 exclude_from_weight_decay=None, dtype=np.float64):
        self.lr, self.wd, self.b1, self.b2, self.eps = learning_rate, weight_decay_rate, beta_1, beta_2, epsilon
        self.exclude = exclude_from_weight_decay
        self.dtype = dtype
        self.m, self.v = {}, {}

    def apply_gradients(self, grads, params):
        """grads, params: {name: array}; params are updated in place and returned."""
        for name, g in grads.items():
            if g is None:
                continue                                                          # :217-218
            g = np.asarray(g, self.dtype)
            p = params[name]
            m = self.m.setdefault(name, np.zeros_like(p, dtype=self.dtype))       # :223-234 zeros
            v = self.v.setdefault(name, np.zeros_like(p, dtype=self.dtype))
            next_m = self.b1 * m + (1.0 - self.b1) * g                            # :241-242
            next_v = self.b2 * v + (1.0 - self.b2) * np.square(g)                 # :243-245
            update = next_m / (np.sqrt(next_v) + self.eps)                        # :247
            if use_weight_decay(name, self.wd, self.exclude):                     # :256-257
                update = update + self.wd * p
            p -= self.lr * update                                                 # :259-261
            self.m[name], self.v[name] = next_m, next_v                           # :263-266
        return params


class Adam:
    """tf.train.AdamOptimizer (xlnet/utils/xlnet_utils.py:195-197)."""

    def __init__(self, learning_rate, beta1=0.9, beta2=0.999, epsilon=1e-8, dtype=np.float64):
        self.lr, self.b1, self.b2, self.eps, self.dtype = learning_rate, beta1, beta2, epsilon, dtype
        self.m, self.v, self.t = {}, {}, 0

    def apply_gradients(self, grads, params, learning_rate=None):
        self.t += 1
        lr = self.lr if learning_rate is None else learning_rate
        lr_t = lr * np.sqrt(1.0 - self.b2 ** self.t) / (1.0 - self.b1 ** self.t)
        for name, g in grads.items():
            g = np.asarray(g, self.dtype)
            p = params[name]
            m = self.m.setdefault(name, np.zeros_like(p, dtype=self.dtype))
            v = self.v.setdefault(name, np.zeros_like(p, dtype=self.dtype))
            m[...] = self.b1 * m + (1.0 - self.b1) * g
            v[...] = self.b2 * v + (1.0 - self.b2) * np.square(g)
            p -= lr_t * m / (np.sqrt(v) + self.eps)
        return params


def gradient_descent(grads, params, learning_rate):
    """tf.train.GradientDescentOptimizer (vgg19/tf-keras-dapple.py:187, 256)."""
    for name, g in grads.items():
        params[name] -= learning_rate * np.asarray(g, params[name].dtype)
    return params


def xlnet_learning_rate(global_step, learning_rate, warmup_steps, train_steps, min_lr_ratio):
    """xlnet/utils/xlnet_utils.py:179-193: linear warm-up while global_step < 1000 (the literal of :192), then
    tf.train.polynomial_decay (power 1, no cycle) from learning_rate to learning_rate * min_lr_ratio over
    train_steps - warmup_steps steps counted from warmup_steps."""
    warmup_lr = float(global_step) / float(warmup_steps) * learning_rate
    end = learning_rate * min_lr_ratio
    decay_steps = train_steps - warmup_steps
    s = min(max(global_step - warmup_steps, 0), decay_steps) if decay_steps > 0 else 0
    decay_lr = (learning_rate - end) * (1.0 - float(s) / decay_steps) + end if decay_steps > 0 else end
    return warmup_lr if global_step < 1000 else decay_lr
