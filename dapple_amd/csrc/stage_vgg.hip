// VGG19 pipeline stage 0: a stack of 3x3 'same' convolutions + ReLU and 2x2 max-pools over NHWC
// fp32 tensors, forward and backward with in-place fp32 weight-gradient accumulation.
//
// Follows vgg19/applications/vgg19_slice_model.py of the reference: layer definitions :135-213
// (keras Conv2D(C,(3,3),activation='relu',padding='same'), MaxPooling2D((2,2),strides=(2,2)),
// HWIO kernels + bias) applied in the order of :280-302.
#include <string.h>

#include "stage.h"

extern "C" int ds_conv3x3_fwd(int dtype, int n, int h, int w, int cin, int cout, const void* x, const void* kernel_hwio,
                              const float* bias, int flags, const void* mask_src, void* y, void* stream);
extern "C" int ds_conv3x3_wgrad(int dtype, int n, int h, int w, int cin, int cout, const void* x, const void* dz,
                                float* dkernel_hwio, void* stream);

namespace {

// out[n,yo,xo,c] = max over the 2x2 window; 4 channels per thread
__global__ __launch_bounds__(256) void maxpool_fwd_kernel(int64_t total4, int H, int W, int C4, const f32x4* __restrict__ x,
                                                         f32x4* __restrict__ y) {
  const int Ho = H / 2, Wo = W / 2;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total4; i += (int64_t)gridDim.x * 256) {
    const int c = (int)(i % C4);
    int64_t t = i / C4;
    const int xo = (int)(t % Wo);
    t /= Wo;
    const int yo = (int)(t % Ho);
    const int64_t n = t / Ho;
    const int64_t base = ((n * H + 2 * yo) * W + 2 * xo) * C4 + c;
    const f32x4 a = x[base], b = x[base + C4], d = x[base + (int64_t)W * C4], e = x[base + (int64_t)W * C4 + C4];
    f32x4 m;
#pragma unroll
    for (int k = 0; k < 4; ++k) m[k] = fmaxf(fmaxf(a[k], b[k]), fmaxf(d[k], e[k]));
    y[i] = m;
  }
}

// The gradient goes to the first maximum of the window (scan order (0,0),(0,1),(1,0),(1,1)); with
// relu_mask it is also zeroed where the pooled input (a ReLU output) is not positive.
__global__ __launch_bounds__(256) void maxpool_bwd_kernel(int64_t total4, int H, int W, int C4, const f32x4* __restrict__ x,
                                                         const f32x4* __restrict__ dy, f32x4* __restrict__ dx, int relu_mask) {
  const int Ho = H / 2, Wo = W / 2;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total4; i += (int64_t)gridDim.x * 256) {
    const int c = (int)(i % C4);
    int64_t t = i / C4;
    const int xo = (int)(t % Wo);
    t /= Wo;
    const int yo = (int)(t % Ho);
    const int64_t n = t / Ho;
    const int64_t base = ((n * H + 2 * yo) * W + 2 * xo) * C4 + c;
    const int64_t o1 = C4, o2 = (int64_t)W * C4, o3 = o2 + C4;
    const f32x4 a = x[base], b = x[base + o1], d = x[base + o2], e = x[base + o3];
    const f32x4 g = dy[i];
    f32x4 ga, gb, gd, ge;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float m = fmaxf(fmaxf(a[k], b[k]), fmaxf(d[k], e[k]));
      const float gg = (relu_mask && !(m > 0.f)) ? 0.f : g[k];
      const bool pa = a[k] == m, pb = !pa && b[k] == m, pd = !pa && !pb && d[k] == m, pe = !pa && !pb && !pd;
      ga[k] = pa ? gg : 0.f; gb[k] = pb ? gg : 0.f; gd[k] = pd ? gg : 0.f; ge[k] = pe ? gg : 0.f;
    }
    dx[base] = ga; dx[base + o1] = gb; dx[base + o2] = gd; dx[base + o3] = ge;
  }
}

// g[i] = y[i] > 0 ? g[i] : 0
__global__ __launch_bounds__(256) void relu_mask_kernel(int64_t total4, const f32x4* __restrict__ y, const f32x4* __restrict__ g,
                                                       f32x4* __restrict__ out) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total4; i += (int64_t)gridDim.x * 256) {
    const f32x4 a = y[i], b = g[i];
    f32x4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) o[k] = a[k] > 0.f ? b[k] : 0.f;
    out[i] = o;
  }
}

// col[p][tap*C + c] = x[p shifted by tap][c] (zero outside the image), padded with zeros to kpad columns
__global__ __launch_bounds__(256) void im2col3x3_kernel(int64_t pixels, int H, int W, int C, int kpad, const float* __restrict__ x,
                                                       float* __restrict__ col) {
  const int64_t total = pixels * kpad;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int k = (int)(i % kpad);
    const int64_t p = i / kpad;
    float v = 0.f;
    if (k < 9 * C) {
      const int tap = k / C, c = k - tap * C;
      const int dy = tap / 3 - 1, dx = tap % 3 - 1;
      const int xx = (int)(p % W), yy = (int)((p / W) % H);
      if ((unsigned)(yy + dy) < (unsigned)H && (unsigned)(xx + dx) < (unsigned)W) v = x[(p + dy * W + dx) * C + c];
    }
    col[i] = v;
  }
}

// wf[(8 - tap), co, c] = w[tap, c, co]: the kernel of the transposed convolution (dgrad)
__global__ __launch_bounds__(256) void conv_flip_kernel(int cin, int cout, const float* __restrict__ w, float* __restrict__ wf) {
  const int total = 9 * cin * cout;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
    const int c = i % cin;
    const int co = (i / cin) % cout;
    const int tf = i / (cin * cout);
    wf[i] = w[((8 - tf) * cin + c) * cout + co];
  }
}

inline int grid_1d(int64_t n) {
  int64_t b = (n + 255) / 256;
  if (b > 256 * 32) b = 256 * 32;
  if (b < 1) b = 1;
  return (int)b;
}

struct Op {
  int cout;  // 0 = pool
  int cin, h, w;  // input extent
  int widx;  // index of the kernel in the weight list (bias = widx + 1), -1 for pools
  size_t in_off, out_off;  // byte offsets into a slot
  size_t in_elems, out_elems;
};

struct VggStage : ds_stage {
  ds_vgg_cfg vc;
  std::vector<Op> ops;
  int N;
  char* stash_base = nullptr;
  size_t slot_bytes = 0;
  char* ws_base = nullptr;
  size_t ws_bytes = 0, ws_g[2], ws_col, ws_fcol, ws_dwpad;
  char* wc_base = nullptr;
  std::vector<float*> wflip;  // per op (conv with dgrad), else null
  float* wpad = nullptr;      // first conv when cin % 32 != 0: [kpad, cout]
  int kpad = 0;
  bool need_dx;

  ~VggStage() override {
    if (stash_base) (void)hipFree(stash_base);
    if (ws_base) (void)hipFree(ws_base);
    if (wc_base) (void)hipFree(wc_base);
  }

  int init() {
    N = vc.batch;
    need_dx = vc.need_input_grad != 0;
    int h = vc.height, w = vc.width, c = vc.in_channels;
    Arena sa;
    size_t cur = sa.reserve((size_t)N * h * w * c * 4);
    size_t max_elems = (size_t)N * h * w * c;
    int block = 1, conv_in_block = 0;
    char name[96];
    for (int i = 0; i < vc.num_ops; ++i) {
      Op o;
      o.cout = vc.ops[i]; o.cin = c; o.h = h; o.w = w; o.in_off = cur; o.in_elems = (size_t)N * h * w * c;
      if (o.cout > 0) {
        ++conv_in_block;
        o.widx = (int)winfo.size();
        snprintf(name, sizeof(name), "block%d_conv%d/kernel", block, conv_in_block);
        winfo.push_back({name, 9 * c, o.cout});
        snprintf(name, sizeof(name), "block%d_conv%d/bias", block, conv_in_block);
        winfo.push_back({name, 1, o.cout});
        c = o.cout;
      } else {
        o.widx = -1;
        h /= 2; w /= 2;
        ++block; conv_in_block = 0;
      }
      o.out_elems = (size_t)N * h * w * c;
      o.out_off = cur = sa.reserve(o.out_elems * 4);
      if (o.out_elems > max_elems) max_elems = o.out_elems;
      ops.push_back(o);
    }
    slot_bytes = sa.used;
    DS_CHECK_HIP(hipMalloc((void**)&stash_base, slot_bytes * vc.stash_slots));
    slot_forwarded.assign(vc.stash_slots, 0);
    // workspace: two gradient buffers, the im2col matrix of a first conv with few channels
    Arena wa;
    ws_g[0] = wa.reserve(max_elems * 4);
    ws_g[1] = wa.reserve(max_elems * 4);
    const Op& first = ops[0];
    if (first.cout > 0 && first.cin % 32 != 0) {
      kpad = ((9 * first.cin + 31) / 32) * 32;
      ws_col = wa.reserve((size_t)N * first.h * first.w * kpad * 4);
      ws_fcol = wa.reserve((size_t)N * first.h * first.w * kpad * 4);  // forward's own patch matrix: backward keeps ws_col
      ws_dwpad = wa.reserve((size_t)kpad * first.cout * 4);
    }
    ws_bytes = wa.used;
    DS_CHECK_HIP(hipMalloc((void**)&ws_base, ws_bytes));
    // compute copies: flipped kernels for dgrad, padded kernel of the first conv
    Arena ca;
    std::vector<size_t> offs(ops.size(), (size_t)-1);
    size_t wpad_off = (size_t)-1;
    for (size_t i = 0; i < ops.size(); ++i) {
      const Op& o = ops[i];
      if (o.cout == 0) continue;
      if (i == 0 && kpad) wpad_off = ca.reserve((size_t)kpad * o.cout * 4);
      if (i > 0 || need_dx) offs[i] = ca.reserve((size_t)9 * o.cin * o.cout * 4);
    }
    if (ca.used) DS_CHECK_HIP(hipMalloc((void**)&wc_base, ca.used));
    wflip.assign(ops.size(), nullptr);
    for (size_t i = 0; i < ops.size(); ++i)
      if (offs[i] != (size_t)-1) wflip[i] = (float*)(wc_base + offs[i]);
    if (wpad_off != (size_t)-1) wpad = (float*)(wc_base + wpad_off);
    return DS_OK;
  }

  size_t workspace_bytes() const override { return ws_bytes; }
  // forward writes its stash slot, its output and its own patch matrix; the rest of the workspace is backward's
  bool overlap_safe() const override { return true; }
  size_t stash_bytes(int slots) const override { return slot_bytes * (size_t)slots; }

  int refresh_weights() override {
    for (size_t i = 0; i < ops.size(); ++i) {
      const Op& o = ops[i];
      if (o.cout == 0) continue;
      if (wflip[i]) {
        hipLaunchKernelGGL(conv_flip_kernel, dim3(grid_1d((int64_t)9 * o.cin * o.cout)), dim3(256), 0, stream, o.cin, o.cout,
                           w[o.widx], wflip[i]);
        DS_CHECK_LAUNCH();
      }
      if (i == 0 && wpad) {
        DS_CHECK_HIP(hipMemsetAsync(wpad, 0, (size_t)kpad * o.cout * 4, stream));
        DS_CHECK_HIP(hipMemcpyAsync(wpad, w[o.widx], (size_t)9 * o.cin * o.cout * 4, hipMemcpyDeviceToDevice, stream));
      }
    }
    return DS_OK;
  }

  int im2col(const Op& o, const float* x, float* col) {
    const int64_t pixels = (int64_t)N * o.h * o.w;
    hipLaunchKernelGGL(im2col3x3_kernel, dim3(grid_1d(pixels * kpad)), dim3(256), 0, stream, pixels, o.h, o.w, o.cin, kpad, x, col);
    DS_CHECK_LAUNCH();
    return DS_OK;
  }

  int forward(int slot, const void* in, const float*, void* out) override {
    ds_prio_scope prio(1);
    char* sp = stash_base + (size_t)slot * slot_bytes;
    DS_CHECK_HIP(hipMemcpyAsync(sp + ops[0].in_off, in, ops[0].in_elems * 4, hipMemcpyDeviceToDevice, stream));
    for (size_t i = 0; i < ops.size(); ++i) {
      const Op& o = ops[i];
      const float* x = (const float*)(sp + o.in_off);
      float* y = (float*)(sp + o.out_off);
      if (o.cout > 0) {
        if (o.cin % 32 == 0) {
          DS_PROPAGATE(ds_conv3x3_fwd(DS_F32, N, o.h, o.w, o.cin, o.cout, x, w[o.widx], w[o.widx + 1],
                                      DS_EPI_BIAS | DS_EPI_RELU, nullptr, y, stream));
        } else {
          float* col = (float*)(ws_base + ws_fcol);
          DS_PROPAGATE(im2col(o, x, col));
          ds_gemm_desc d;
          memset(&d, 0, sizeof(d));
          d.dtype = DS_F32; d.a_major = DS_K_MAJOR; d.b_major = DS_MN_MAJOR;
          d.m = N * o.h * o.w; d.n = o.cout; d.k = kpad; d.lda = kpad; d.ldb = o.cout; d.ldc = o.cout;
          d.batch = 1; d.batch_inner = 1; d.flags = DS_EPI_BIAS | DS_EPI_RELU; d.alpha = 1.f;
          d.a = col; d.b = wpad; d.c = y; d.bias = w[o.widx + 1];
          DS_PROPAGATE(ds_gemm(&d, stream));
        }
      } else {
        const int64_t total4 = (int64_t)o.out_elems / 4;
        hipLaunchKernelGGL(maxpool_fwd_kernel, dim3(grid_1d(total4)), dim3(256), 0, stream, total4, o.h, o.w, o.cin / 4,
                           (const f32x4*)x, (f32x4*)y);
        DS_CHECK_LAUNCH();
      }
    }
    const Op& last = ops.back();
    DS_CHECK_HIP(hipMemcpyAsync(out, sp + last.out_off, last.out_elems * 4, hipMemcpyDeviceToDevice, stream));
    return DS_OK;
  }

  int backward(int slot, const void* d_out, void* d_in) override {
    ds_prio_scope prio(3);  // the chain every later pass waits on
    char* sp = stash_base + (size_t)slot * slot_bytes;
    const float* gout = (const float*)d_out;
    int cur = -1;         // which workspace buffer gout lives in (-1: the caller's d_out)
    bool masked = false;  // whether gout already carries the ReLU mask of the conv that produced this tensor
    auto other = [](int c) { return c == 0 ? 1 : 0; };
    for (int i = (int)ops.size() - 1; i >= 0; --i) {
      const Op& o = ops[i];
      const float* x = (const float*)(sp + o.in_off);
      const float* y = (const float*)(sp + o.out_off);
      const bool want_gin = i > 0 || (need_dx && d_in);
      const bool below_is_conv = i > 0 && ops[i - 1].cout > 0;
      if (o.cout > 0) {
        if (!masked) {
          const int t = other(cur);
          float* gm = (float*)(ws_base + ws_g[t]);
          const int64_t total4 = (int64_t)o.out_elems / 4;
          hipLaunchKernelGGL(relu_mask_kernel, dim3(grid_1d(total4)), dim3(256), 0, stream, total4, (const f32x4*)y,
                             (const f32x4*)gout, (f32x4*)gm);
          DS_CHECK_LAUNCH();
          gout = gm;
          cur = t;
        }
        const int pixels = N * o.h * o.w;
        DS_PROPAGATE(ds_colsum_accum(DS_F32, pixels, o.cout, gout, o.cout, g[o.widx + 1], stream));
        if (o.cin % 32 == 0) {
          DS_PROPAGATE(ds_conv3x3_wgrad(DS_F32, N, o.h, o.w, o.cin, o.cout, x, gout, g[o.widx], stream));
        } else {
          float* col = (float*)(ws_base + ws_col);
          float* dwpad = (float*)(ws_base + ws_dwpad);
          DS_PROPAGATE(im2col(o, x, col));
          DS_CHECK_HIP(hipMemsetAsync(dwpad, 0, (size_t)kpad * o.cout * 4, stream));
          ds_gemm_desc d;
          memset(&d, 0, sizeof(d));
          d.dtype = DS_F32; d.a_major = DS_MN_MAJOR; d.b_major = DS_MN_MAJOR;
          d.m = kpad; d.n = o.cout; d.k = pixels; d.lda = kpad; d.ldb = o.cout; d.ldc = o.cout;
          d.batch = 1; d.batch_inner = 1; d.flags = DS_EPI_ACCUM; d.alpha = 1.f;
          d.a = col; d.b = gout; d.c = dwpad;
          DS_PROPAGATE(ds_gemm_splitk(&d, 256, stream));
          DS_PROPAGATE(ds_grad_accumulate(g[o.widx], dwpad, (size_t)9 * o.cin * o.cout, DS_F32, stream));
        }
        if (!want_gin) break;
        // dgrad = the same convolution of gout with the flipped kernel; the ReLU mask of the conv below is fused in
        const int t = other(cur);
        float* gin = (i == 0) ? (float*)d_in : (float*)(ws_base + ws_g[t]);
        DS_PROPAGATE(ds_conv3x3_fwd(DS_F32, N, o.h, o.w, o.cout, o.cin, gout, wflip[i], nullptr, below_is_conv ? DS_EPI_MASK : 0,
                                    below_is_conv ? (const void*)x : nullptr, gin, stream));
        gout = gin;
        cur = t;
        masked = below_is_conv;
      } else {
        if (!want_gin) break;
        const int t = other(cur);
        float* gin = (i == 0) ? (float*)d_in : (float*)(ws_base + ws_g[t]);
        const int64_t total4 = (int64_t)o.out_elems / 4;
        hipLaunchKernelGGL(maxpool_bwd_kernel, dim3(grid_1d(total4)), dim3(256), 0, stream, total4, o.h, o.w, o.cin / 4,
                           (const f32x4*)x, (const f32x4*)gout, (f32x4*)gin, below_is_conv ? 1 : 0);
        DS_CHECK_LAUNCH();
        gout = gin;
        cur = t;
        masked = below_is_conv;
      }
    }
    return DS_OK;
  }
};

}  // namespace

extern "C" int ds_vgg_stage_create(const ds_vgg_cfg* c, void* stream, ds_stage** out) {
  DS_CHECK_ARG(c != nullptr && out != nullptr, "ds_vgg_stage_create: null argument");
  *out = nullptr;
  DS_CHECK_ARG(c->dtype == DS_F32, "ds_vgg_stage_create: only fp32 is built (dtype %d)", c->dtype);
  DS_CHECK_ARG(c->batch > 0 && c->height > 0 && c->width > 0 && c->in_channels > 0, "ds_vgg_stage_create: non-positive input shape");
  DS_CHECK_ARG(c->num_ops > 0 && c->num_ops <= 40, "ds_vgg_stage_create: num_ops %d outside [1,40]", c->num_ops);
  DS_CHECK_ARG(c->stash_slots >= 1, "ds_vgg_stage_create: stash_slots must be >= 1");
  int h = c->height, w = c->width, ch = c->in_channels;
  for (int i = 0; i < c->num_ops; ++i) {
    if (c->ops[i] > 0) {
      DS_CHECK_ARG(i == 0 || ch % 32 == 0, "ds_vgg_stage_create: conv %d has %d input channels; only the first conv may have a count that is not a multiple of 32", i, ch);
      DS_CHECK_ARG(c->ops[i] % 4 == 0, "ds_vgg_stage_create: conv %d output channels (%d) must be a multiple of 4", i, c->ops[i]);
      DS_CHECK_ARG(((int64_t)c->batch * h * w) % 32 == 0, "ds_vgg_stage_create: batch*h*w (%lld) at conv %d must be a multiple of 32",
                   (long long)c->batch * h * w, i);
      if (i == 0 && ch % 32 != 0) DS_CHECK_ARG(!c->need_input_grad, "ds_vgg_stage_create: no input gradient through a first conv with %d channels", ch);
      ch = c->ops[i];
    } else {
      DS_CHECK_ARG(c->ops[i] == 0, "ds_vgg_stage_create: op %d is negative", i);
      DS_CHECK_ARG(h % 2 == 0 && w % 2 == 0 && ch % 4 == 0, "ds_vgg_stage_create: pool %d needs even height/width and channels %% 4 == 0", i);
      h /= 2; w /= 2;
    }
  }
  VggStage* s = new VggStage();
  memset(&s->cfg, 0, sizeof(s->cfg));
  s->cfg.kind = DS_STAGE_VGG19;
  s->cfg.dtype = c->dtype;
  s->cfg.stash_slots = c->stash_slots;
  s->vc = *c;
  s->stream = (hipStream_t)stream;
  const int rc = s->init();
  if (rc != DS_OK) { delete s; return rc; }
  *out = s;
  return DS_OK;
}

// unit entry points -------------------------------------------------------------------------
extern "C" int ds_vgg_stage_read_activation(ds_stage* h, int slot, int op, float* dst, size_t dst_elems) {
  DS_CHECK_ARG(h != nullptr && dst != nullptr, "ds_vgg_stage_read_activation: null argument");
  DS_CHECK_ARG(h->cfg.kind == DS_STAGE_VGG19, "ds_vgg_stage_read_activation: not a VGG stage");
  VggStage* s = static_cast<VggStage*>(h);
  DS_CHECK_ARG(slot >= 0 && slot < s->vc.stash_slots, "ds_vgg_stage_read_activation: slot %d out of range", slot);
  DS_CHECK_ARG(op >= 0 && op < (int)s->ops.size(), "ds_vgg_stage_read_activation: op %d out of range [0,%d)", op, (int)s->ops.size());
  if (!s->slot_forwarded[slot]) {
    ds_set_error("ds_vgg_stage_read_activation: slot %d holds no forwarded micro-batch", slot);
    return DS_ESTATE;
  }
  const Op& o = s->ops[op];
  DS_CHECK_ARG(dst_elems == o.out_elems, "ds_vgg_stage_read_activation: op %d has %zu elements, the buffer %zu", op, o.out_elems, dst_elems);
  DS_CHECK_HIP(hipMemcpyAsync(dst, s->stash_base + (size_t)slot * s->slot_bytes + o.out_off, o.out_elems * 4, hipMemcpyDeviceToDevice,
                              s->stream));
  return DS_OK;
}

extern "C" int ds_maxpool2x2_fwd(int n, int h, int w, int c, const float* x, float* y, void* stream) {
  DS_CHECK_ARG(n > 0 && h > 0 && w > 0 && c > 0 && h % 2 == 0 && w % 2 == 0 && c % 4 == 0 && x && y,
               "ds_maxpool2x2_fwd: needs even h, w, c %% 4 == 0 and non-null pointers");
  const int64_t total4 = (int64_t)n * (h / 2) * (w / 2) * c / 4;
  hipLaunchKernelGGL(maxpool_fwd_kernel, dim3(grid_1d(total4)), dim3(256), 0, (hipStream_t)stream, total4, h, w, c / 4,
                     (const f32x4*)x, (f32x4*)y);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_maxpool2x2_bwd(int n, int h, int w, int c, const float* x, const float* dy, float* dx, int relu_mask, void* stream) {
  DS_CHECK_ARG(n > 0 && h > 0 && w > 0 && c > 0 && h % 2 == 0 && w % 2 == 0 && c % 4 == 0 && x && dy && dx,
               "ds_maxpool2x2_bwd: needs even h, w, c %% 4 == 0 and non-null pointers");
  const int64_t total4 = (int64_t)n * (h / 2) * (w / 2) * c / 4;
  hipLaunchKernelGGL(maxpool_bwd_kernel, dim3(grid_1d(total4)), dim3(256), 0, (hipStream_t)stream, total4, h, w, c / 4,
                     (const f32x4*)x, (const f32x4*)dy, (f32x4*)dx, relu_mask);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_conv3x3_flip(int cin, int cout, const float* kernel_hwio, float* flipped, void* stream) {
  DS_CHECK_ARG(cin > 0 && cout > 0 && kernel_hwio && flipped, "ds_conv3x3_flip: bad argument");
  hipLaunchKernelGGL(conv_flip_kernel, dim3(grid_1d((int64_t)9 * cin * cout)), dim3(256), 0, (hipStream_t)stream, cin, cout,
                     kernel_hwio, flipped);
  DS_CHECK_LAUNCH();
  return DS_OK;
}
