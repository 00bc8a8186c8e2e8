"""VGG19 stage-0 parity through the C ABI: implicit-GEMM conv fwd / dgrad / wgrad, max-pool, and
the whole stage under the 2S-1 schedule variant, against the fp64 CPU oracle (fp32: 1e-4 relative)."""
import numpy as np
import pytest
import torch

from dapple_amd import ops, runtime, synthetic
from oracle import vgg as ov
from util import assert_close, dev

pytestmark = pytest.mark.gpu
TOL = 1e-4


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


@pytest.mark.parametrize("n,h,w,cin,cout", [(2, 8, 8, 32, 32), (2, 8, 8, 64, 128), (1, 6, 10, 32, 64), (3, 5, 7, 96, 36),
                                           (2, 14, 14, 128, 256)])
def test_conv_fwd_dgrad_wgrad(n, h, w, cin, cout):
    r = rng(n * h + cin + cout)
    x = dev(r.standard_normal((n, h, w, cin)).astype(np.float32))
    k = dev((r.standard_normal((3, 3, cin, cout)) * 0.1).astype(np.float32))
    b = dev(r.standard_normal(cout).astype(np.float32))
    dy = dev(r.standard_normal((n, h, w, cout)).astype(np.float32))
    x64, k64, b64 = x.cpu().double().requires_grad_(True), k.cpu().double().requires_grad_(True), b.cpu().double().requires_grad_(True)
    y64 = ov.conv3x3_relu(x64, k64, b64)
    y = ops.conv3x3(x, k, b, relu=True)
    assert_close(y, y64, TOL, "conv fwd")
    dx64, dk64, db64 = torch.autograd.grad(y64, [x64, k64, b64], dy.cpu().double())
    # backward the way the stage does it: mask, then conv with the flipped kernel, then wgrad
    dz = torch.where(y > 0, dy, torch.zeros_like(dy))
    if cout % 32 == 0:
        dx = ops.conv3x3(dz, ops.conv3x3_flip(k))
        assert_close(dx, dx64, TOL, "conv dgrad")
    if (n * h * w) % 32 == 0:
        dk = torch.ones_like(k)
        ops.conv3x3_wgrad(x, dz, dk)
        assert_close(dk, dk64 + 1, TOL, "conv wgrad (accumulates)")


def test_conv_mask_epilogue():
    r = rng(5)
    x = dev(r.standard_normal((2, 4, 4, 32)).astype(np.float32))
    k = dev((r.standard_normal((3, 3, 32, 32)) * 0.1).astype(np.float32))
    m = dev(r.standard_normal((2, 4, 4, 32)).astype(np.float32))
    y = ops.conv3x3(x, k, mask_src=m)
    ref = ops.conv3x3(x, k)
    assert torch.equal(y, torch.where(m > 0, ref, torch.zeros_like(ref)))


def test_conv_rejects_bad_channels():
    x = torch.zeros(1, 4, 4, 3, device="cuda")
    k = torch.zeros(3, 3, 3, 8, device="cuda")
    with pytest.raises(ValueError, match="multiple of 32"):
        ops.conv3x3(x, k)


def test_maxpool_fwd_bwd():
    r = rng(9)
    x = dev(r.standard_normal((2, 6, 8, 8)).astype(np.float32))
    x[0, 0, 0, 0] = x[0, 0, 1, 0] = x[0, 1, 0, 0] = x[0, 1, 1, 0] = 0.5      # a 4-way tie: first position wins
    dy = dev(r.standard_normal((2, 3, 4, 8)).astype(np.float32))
    y = ops.maxpool2x2(x)
    x64 = x.cpu().double().requires_grad_(True)
    y64 = ov.max_pool_2x2(x64)
    assert torch.equal(y.cpu().double(), y64.detach())
    (dx64,) = torch.autograd.grad(y64, x64, dy.cpu().double())
    dx = ops.maxpool2x2_bwd(x, dy)
    assert dx[0, 0, 0, 0] == dy[0, 0, 0, 0] and dx[0, 0, 1, 0] == 0 and dx[0, 1, 0, 0] == 0
    dx64[0, :2, :2, 0] = 0
    dx64[0, 0, 0, 0] = dy[0, 0, 0, 0].item()        # torch's tie rule may differ from the first-maximum rule
    assert torch.equal(dx.cpu().double(), dx64)
    dxm = ops.maxpool2x2_bwd(x, dy, relu_mask=True)
    want = ops.maxpool2x2_bwd(x, dy) * (x > 0)
    assert torch.equal(dxm, want)


def run_stage(channels, n, h, w, cin, M, K, variant="2S-1", need_dx=False, odtype=torch.float64, seed=0, perturb=True,
              grad_tol=TOL):
    layers = synthetic.vgg_layers(channels)
    w_np = synthetic.vgg_weights(synthetic.SEED_WEIGHT + seed, layers, cin, perturb=perturb)
    xs_np = synthetic.vgg_inputs(synthetic.SEED_INPUT + seed, M, n, h, w, cin)
    stage = runtime.vgg_stage(layers, n, h, w, cin, stash_slots=K, need_input_grad=need_dx)
    stage.bind(w_np)
    dys_np = synthetic.upstream_grads(synthetic.SEED_GRAD + seed, M, stage.out_shape)
    xs, dys = [dev(x) for x in xs_np], [dev(d) for d in dys_np]
    outs = [torch.empty(stage.out_shape, device="cuda") for _ in range(M)]
    dxs = [torch.empty_like(x) for x in xs] if need_dx else None
    # stage 0 of S where 2S-1-0 == K (variant of vgg19/tf-keras-dapple.py:292) or S-0 == K
    S = (K + 1) // 2 if variant == "2S-1" else K
    rt = runtime.StageRuntime(stage, 0, S, M, variant=variant, needs_input_grad=need_dx)
    rt.step(xs, dys, outs, dxs)
    stage.sync()
    w_t = ov.to_torch(w_np, odtype, requires_grad=True)
    acc = {}
    for j in range(M):
        out, dx, dw = ov.stage_vjp(xs[j].cpu().to(odtype), w_t, dys[j].cpu().to(odtype), layers, need_input_grad=need_dx)
        assert_close(outs[j], out, TOL, "output mb%d" % j)
        if need_dx:
            assert_close(dxs[j], dx, TOL, "input grad mb%d" % j)
        for k_, g in dw.items():
            acc[k_] = g.clone() if k_ not in acc else acc[k_] + g
    for name in stage.weight_names:
        assert_close(stage.grads[name], acc[name], grad_tol, "accumulated grad " + name)
    stage.close()


def test_stage_small_first_conv_3_channels():
    run_stage([32, 32, None, 64, 64, None, 64], n=2, h=16, w=16, cin=3, M=4, K=3)


def test_stage_small_with_input_grad_and_pool_last():
    run_stage([32, None, 64, None], n=2, h=8, w=16, cin=32, M=3, K=2, variant="S", need_dx=True, seed=1)


def test_stage_vgg19_stack_full_depth_reduced_batch():
    # BASELINE configs[1] topology and image size (16 convs, 4 pools, 224x224x3), micro-batch 8, one micro-batch.
    # Outputs are held to 1e-4.  Gradients through 16 ReLUs and 4 max-pools over ~10^8 activations are
    # not: an fp32 pre-activation within rounding of zero (or two window entries within rounding of each
    # other) takes the other branch than the fp64 oracle at a handful of positions, and each such flip
    # moves a whole gradient entry.  Measured: 3e-4 after block5, 5e-3 below pool4, never growing with
    # depth otherwise.  The per-layer test below holds every backward kernel to 1e-4 at the real layer
    # shapes, and the linearity test holds the full-depth backward to 1e-4 against itself.
    c = synthetic.CONFIGS["vgg19_stage0"]
    run_stage([co for _, co in c["layers"]], n=8, h=c["height"], w=c["width"], cin=c["in_channels"], M=1, K=3,
              odtype=torch.float64, seed=c["index"], perturb=False, grad_tol=3e-2)


def _forced_branch_case(channels, n, h, w, cin, seed, perturb, tol):
    """One micro-batch through the stage; the oracle walks the branches the GPU took (ReLU masks = stashed activation > 0,
    pool picks = argmax of the stashed pool input) in fp64: what is left between the two is rounding."""
    layers = synthetic.vgg_layers(channels)
    w_np = synthetic.vgg_weights(synthetic.SEED_WEIGHT + seed, layers, cin, perturb=perturb)
    x_np = synthetic.vgg_inputs(synthetic.SEED_INPUT + seed, 1, n, h, w, cin)[0]
    stage = runtime.vgg_stage(layers, n, h, w, cin, stash_slots=1)
    stage.bind(w_np)
    dy_np = synthetic.upstream_grads(synthetic.SEED_GRAD + seed, 1, stage.out_shape)[0]
    x, dy = dev(x_np), dev(dy_np)
    out = torch.empty(stage.out_shape, device="cuda")
    stage.forward(0, x, out)
    masks, picks = {}, {}
    hh, ww, cc = h, w, cin
    prev = x
    for i, (name, cout) in enumerate(layers):
        if cout is None:
            win = prev.reshape(n, hh // 2, 2, ww // 2, 2, cc).permute(0, 1, 3, 5, 2, 4).reshape(n, hh // 2, ww // 2, cc, 4)
            picks[name] = win.argmax(-1).cpu()
            hh, ww = hh // 2, ww // 2
        else:
            cc = cout
        prev = stage.read_activation(0, i, (n, hh, ww, cc))
        if cout is not None:
            masks[name] = (prev > 0).cpu()
    stage.backward(0, dy)
    stage.sync()
    w_t = ov.to_torch(w_np, torch.float64, requires_grad=True)
    o_ref, _, dw = ov.stage_vjp_forced_branches(x.cpu().double(), w_t, dy.cpu().double(), layers, masks, picks)
    assert_close(out, o_ref, tol, "output")
    for name in stage.weight_names:
        assert_close(stage.grads[name], dw[name], tol, "grad " + name)
    stage.close()


def test_forced_branch_oracle_small():
    _forced_branch_case([32, 32, None, 64, 64, None, 64], n=2, h=16, w=16, cin=3, seed=11, perturb=True, tol=TOL)


def test_config1_full_size_along_the_gpus_own_branches():
    """BASELINE configs[1] at its stated size - conv1_1 .. conv5_4, 4 pools, 32 images of 224 x 224 x 3 - one micro-batch:
    outputs and all 32 weight / bias gradients at 1e-4 against the fp64 oracle walking the branches the GPU took (the
    accumulation over 4 micro-batches is the stage-independent sum the smaller cases and the linearity test cover)."""
    c = synthetic.CONFIGS["vgg19_stage0"]
    _forced_branch_case([co for _, co in c["layers"]], n=c["micro_batch"], h=c["height"], w=c["width"], cin=c["in_channels"],
                        seed=c["index"], perturb=False, tol=TOL)


@pytest.mark.parametrize("n,h,w,cin,cout", [(8, 224, 224, 64, 64), (8, 28, 28, 256, 512), (32, 14, 14, 512, 512)])
def test_conv_backward_at_real_layer_shapes(n, h, w, cin, cout):
    # one layer has no downstream discontinuity: the mask is taken from the GPU forward on both sides
    r = rng(cin + h)
    x = dev(r.standard_normal((n, h, w, cin)).astype(np.float32))
    k = dev((r.standard_normal((3, 3, cin, cout)) * np.sqrt(2.0 / (9 * cin))).astype(np.float32))
    dz = dev(r.standard_normal((n, h, w, cout)).astype(np.float32))
    x_t = x.cpu().requires_grad_(True)
    k_t = k.cpu().requires_grad_(True)
    y = torch.nn.functional.conv2d(x_t.permute(0, 3, 1, 2), k_t.permute(3, 2, 0, 1), padding=1).permute(0, 2, 3, 1)
    dx_ref, dk_ref = torch.autograd.grad(y, [x_t, k_t], dz.cpu())
    assert_close(ops.conv3x3(x, k), y, TOL, "fwd")
    assert_close(ops.conv3x3(dz, ops.conv3x3_flip(k)), dx_ref, TOL, "dgrad")
    dk = torch.zeros_like(k)
    ops.conv3x3_wgrad(x, dz, dk)
    assert_close(dk, dk_ref, TOL, "wgrad")


def test_full_depth_backward_is_linear_in_the_upstream_gradient():
    # with the forward (hence every ReLU mask and pool argmax) fixed in the stash, backward is linear:
    # grads(a*dy1 + dy2) == a*grads(dy1) + grads(dy2), at the full 16-conv depth and 224x224 images
    c = synthetic.CONFIGS["vgg19_stage0"]
    layers, n = c["layers"], 8
    stage = runtime.vgg_stage(layers, n, 224, 224, 3, stash_slots=1)
    stage.bind(synthetic.vgg_weights(7, layers, 3))
    x = dev(synthetic.vgg_inputs(8, 1, n, 224, 224, 3)[0])
    d1, d2 = [dev(d) for d in synthetic.upstream_grads(9, 2, stage.out_shape)]
    out = torch.empty(stage.out_shape, device="cuda")
    res = []
    for dy in (d1, d2, 0.5 * d1 + d2):
        stage.zero_grads()
        stage.forward(0, x, out)
        stage.backward(0, dy.contiguous(), None)
        stage.sync()
        res.append(stage.flat_grads.clone())
    assert_close(res[2], 0.5 * res[0] + res[1], TOL, "linearity")
    stage.close()
