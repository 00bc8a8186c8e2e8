"""CPU restatement of the reference's VGG19 stage-0 slice. TEST INFRASTRUCTURE ONLY.

Follows vgg19/applications/vgg19_slice_model.py:135-213 (layer definitions: keras
Conv2D(C, (3,3), activation='relu', padding='same'), MaxPooling2D((2,2), strides=(2,2)),
channels_last, kernel HWIO [3,3,Cin,Cout] + bias) and :274-309 (the order they are applied
in on a stage-0 replica).  Tensors are NHWC like the reference; torch's NCHW conv is
reached by permutation.  Backward is torch.autograd.

Pins (tests/test_oracle_vgg.py): conv vs a brute-force 7-deep loop; 'same' padding = 1;
max-pool vs brute force; ReLU gradient 0 at exactly 0; parameter counts vs
profiling_results/vgg-19-pbs-32.txt of the reference; stage_vjp_forced_branches vs stage_vjp with the
branches it took itself, and vs brute force on a case with flipped branches; the classification block and both
losses of head_forward / head_loss vs scalar loops, torch's cross_entropy and the closed form of the as-written loss.
"""
import torch

# (name, out_channels) or (name, None) for a pool, in application order (:280-302)
VGG19_STAGE0_15_1 = [
    ("block1_conv1", 64), ("block1_conv2", 64), ("block1_pool", None),
    ("block2_conv1", 128), ("block2_conv2", 128), ("block2_pool", None),
    ("block3_conv1", 256), ("block3_conv2", 256), ("block3_conv3", 256), ("block3_conv4", 256), ("block3_pool", None),
    ("block4_conv1", 512), ("block4_conv2", 512), ("block4_conv3", 512), ("block4_conv4", 512), ("block4_pool", None),
    ("block5_conv1", 512), ("block5_conv2", 512),
]
# BASELINE configs[1]: conv1_1..conv5_4 (16 convs, 4 pools)
VGG19_CONV_STACK = VGG19_STAGE0_15_1 + [("block5_conv3", 512), ("block5_conv4", 512)]


def conv3x3_relu(x, kernel, bias):
    """keras Conv2D(3x3, 'same', relu) on NHWC x with HWIO kernel."""
    y = torch.nn.functional.conv2d(x.permute(0, 3, 1, 2), kernel.permute(3, 2, 0, 1), bias, stride=1, padding=1)
    return torch.relu(y).permute(0, 2, 3, 1)


def max_pool_2x2(x):
    """keras MaxPooling2D((2,2), strides=(2,2)), 'valid'."""
    return torch.nn.functional.max_pool2d(x.permute(0, 3, 1, 2), 2, 2).permute(0, 2, 3, 1)


def stage_forward(x, w, layers):
    for name, cout in layers:
        if cout is None:
            x = max_pool_2x2(x)
        else:
            x = conv3x3_relu(x, w[name + "/kernel"], w[name + "/bias"])
    return x


def to_torch(weights, dtype=torch.float64, requires_grad=False):
    return {k: torch.as_tensor(v).to(dtype).clone().requires_grad_(requires_grad) for k, v in weights.items()}


def stage_vjp(x, w, d_out, layers, need_input_grad=False):
    """tf.gradients(ys=out, xs=vars (+ input), grad_ys=d_out): (out, d_x or None, {name: d_w})."""
    names = sorted(w)
    if need_input_grad:
        x = x.clone().requires_grad_(True)
    out = stage_forward(x, w, layers)
    xs = ([x] if need_input_grad else []) + [w[n] for n in names]
    grads = torch.autograd.grad(out, xs, grad_outputs=d_out, allow_unused=True)
    off = 1 if need_input_grad else 0
    return out.detach(), (grads[0] if need_input_grad else None), {n: g for n, g in zip(names, grads[off:]) if g is not None}


def branches_of(x, w, layers):
    """The discrete choices of a forward pass: per conv the ReLU mask (bool, NHWC), per pool the index 0..3 of the
    window entry that is the maximum (row-major inside the 2x2 window, first maximum on ties)."""
    masks, picks = {}, {}
    for name, cout in layers:
        if cout is None:
            n, h, wd, c = x.shape
            win = x.reshape(n, h // 2, 2, wd // 2, 2, c).permute(0, 1, 3, 5, 2, 4).reshape(n, h // 2, wd // 2, c, 4)
            picks[name] = win.argmax(-1)
            x = max_pool_2x2(x)
        else:
            x = conv3x3_relu(x, w[name + "/kernel"], w[name + "/bias"])
            masks[name] = x > 0
    return masks, picks


def stage_vjp_forced_branches(x, w, d_out, layers, masks, picks, need_input_grad=False):
    """stage_vjp along GIVEN branches: ReLU is multiplication by masks[name], max-pool picks window entry picks[name].
    ReLU and max-pool are the only discontinuities of the stage; a device pass in fp32 takes the other branch than an
    fp64 pass wherever a pre-activation (or the gap between two window entries) is within rounding of zero, and a
    flipped branch moves a whole gradient entry.  With the branches of the device pass forced, what is left is smooth
    (linear in each weight), and fp64 gives the exact derivative of the function the device actually evaluated."""
    names = sorted(w)
    if need_input_grad:
        x = x.clone().requires_grad_(True)
    h = x
    for name, cout in layers:
        if cout is None:
            n, hh, wd, c = h.shape
            win = h.reshape(n, hh // 2, 2, wd // 2, 2, c).permute(0, 1, 3, 5, 2, 4).reshape(n, hh // 2, wd // 2, c, 4)
            h = win.gather(-1, picks[name].unsqueeze(-1)).squeeze(-1)
        else:
            z = torch.nn.functional.conv2d(h.permute(0, 3, 1, 2), w[name + "/kernel"].permute(3, 2, 0, 1), w[name + "/bias"],
                                           stride=1, padding=1).permute(0, 2, 3, 1)
            h = z * masks[name].to(z.dtype)
    xs = ([x] if need_input_grad else []) + [w[n] for n in names]
    grads = torch.autograd.grad(h, xs, grad_outputs=d_out, allow_unused=True)
    off = 1 if need_input_grad else 0
    return h.detach(), (grads[0] if need_input_grad else None), {n: g for n, g in zip(names, grads[off:]) if g is not None}


# ---------------------------------------------------------------------------------------- last stage: classification block
def head_forward(x, hw):
    """vgg19_slice_model.py:217-220 applied at :342-347: Flatten (the caller passes [batch, features]), fc1 and fc2 =
    Dense(4096, relu), predictions = Dense(classes, softmax); kernels in keras' [in, out] layout."""
    h1 = torch.relu(x @ hw["fc1/kernel"] + hw["fc1/bias"])
    h2 = torch.relu(h1 @ hw["fc2/kernel"] + hw["fc2/bias"])
    return torch.softmax(h2 @ hw["predictions/kernel"] + hw["predictions/bias"], -1)


def keras_categorical_crossentropy(target, output, epsilon=1e-7):
    """keras.backend.categorical_crossentropy(target, output) of the TensorFlow backend for probabilities
    (from_logits=False), restated from its published definition (keras is not vendored in the reference):
    output /= reduce_sum(output, -1, keepdims); output = clip(output, eps, 1 - eps); -reduce_sum(target * log(output), -1)."""
    output = output / output.sum(-1, keepdim=True)
    output = torch.clamp(output, epsilon, 1.0 - epsilon)
    return -(target * torch.log(output)).sum(-1)


def head_loss(probs, labels, mode="as_written"):
    """vgg19_slice_model.py:354-355.  "as_written": K.categorical_crossentropy(x, label) exactly as called - the softmax
    output lands in the `target` slot and the [batch, 1] float label column in the `output` slot - then reduce_mean.
    "sparse_ce": mean of -log probs[label] with the label as a class index."""
    if mode == "as_written":
        return keras_categorical_crossentropy(probs, labels.reshape(-1, 1).to(probs.dtype)).mean()
    idx = labels.to(torch.int64)
    return -torch.log(probs[torch.arange(probs.shape[0]), idx]).mean()
