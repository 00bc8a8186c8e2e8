// GNMT encoder pipeline stage: embedding lookup, one bidirectional LSTM layer, uni-directional LSTM
// layers (residual from the third layer on), forward and BPTT backward, fp32.
//
// Follows gnmt/nmt/gnmt_model.py:61-221 (DAPPLE branch) and gnmt/nmt/model_helper.py:399-456 of the
// reference; the cell is TensorFlow's BasicLSTMCell: gates = [x, h] @ kernel[in+U, 4U] + bias, gate
// order i, j, f, o, c' = c*sigmoid(f + forget_bias) + sigmoid(i)*tanh(j), h' = tanh(c')*sigmoid(o).
// Without lengths dynamic_rnn is a plain scan.  With source_sequence_length (gnmt_model.py:103, 223-227) a
// step t >= length[b] emits zeros - also from a residual cell, whose wrapped output is what gets replaced - and
// keeps the state; the backward direction starts from the zero state at t = length[b] - 1.  Here such a
// step stores h = c = y = 0 (in either scan order it lies outside the run of live steps, which therefore
// starts from zeros) and backward gives it zero gate gradients and passes no state gradient on.
//
// Per layer: the input half of the gates for all T steps is ONE GEMM [T*B, in] x [in, 4U] (+bias);
// each step then adds h[t-1] @ Wh (a [B, U] x [U, 4U] GEMM whose epilogue adds the precomputed
// half in place) and runs the fused cell kernel.  Backward walks the steps in reverse with the cell
// backward kernel and dh = dgates @ Wh^T, then finishes with three big GEMMs over all steps:
// dX = dG @ Wx^T, dWx += X^T dG, dWh += Hprev^T dG.
#include <stdlib.h>
#include <string.h>

#include "stage.h"

namespace {

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

// table rows -> time-major activations: x[(t*B + b), :] = table[ids[b*T + t], :]
__global__ __launch_bounds__(256) void gnmt_embed_fwd_kernel(int B, int T, int U, int vocab, const int32_t* __restrict__ ids,
                                                            const float* __restrict__ table, float* __restrict__ x) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= B * T) return;
  const int t = row / B, b = row % B;
  int id = ids[b * T + t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const f32x4* src = reinterpret_cast<const f32x4*>(table + (int64_t)id * U);
  f32x4* dst = reinterpret_cast<f32x4*>(x + (int64_t)row * U);
  for (int c = threadIdx.x & 63; c < U / 4; c += 64) dst[c] = src[c];
}

__global__ __launch_bounds__(256) void gnmt_embed_bwd_kernel(int B, int T, int U, int vocab, const int32_t* __restrict__ ids,
                                                            const float* __restrict__ dx, float* __restrict__ dtable) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= B * T) return;
  const int t = row / B, b = row % B;
  int id = ids[b * T + t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  for (int c = threadIdx.x & 63; c < U; c += 64) atomicAdd(dtable + (int64_t)id * U + c, dx[(int64_t)row * U + c]);
}

// One time step of the cell.  gates [B,4U] holds the pre-activations (bias included) and is
// overwritten with the activated gates (sigmoid(i), tanh(j), sigmoid(f + forget_bias), sigmoid(o));
// h is written with row stride ldh, and y = h + x_res when the cell has a residual connection.
// part (nullable) [nparts][B][4U]: partial sums of the recurrent product h_{t-1} Wh, one per slice of the reduction,
// added to the pre-activations here - the product is split so that every CU has work, and summing the slices where
// they are consumed costs a few reads where atomic adds from the product's epilogue cost as much as the product.
__global__ __launch_bounds__(256) void lstm_cell_fwd_kernel(int B, int U, float forget_bias, float* __restrict__ gates,
                                                           const float* __restrict__ c_prev, float* __restrict__ c,
                                                           float* __restrict__ h, int ldh, const float* __restrict__ x_res,
                                                           int ldx, float* __restrict__ y, int ldy,
                                                           const int32_t* __restrict__ len, int t, const float* __restrict__ part,
                                                           int nparts) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= B * U) return;
  const int b = idx / U, u = idx % U;
  if (len && t >= len[b]) {  // past the end of sequence b
    c[idx] = 0.f;
    h[(int64_t)b * ldh + u] = 0.f;
    if (y) y[(int64_t)b * ldy + u] = 0.f;
    return;
  }
  float* g = gates + (int64_t)b * 4 * U;
  float gi = g[u], gj = g[U + u], gf = g[2 * U + u], go = g[3 * U + u];
  const float cp = c_prev ? c_prev[idx] : 0.f;
  const float xr = y ? x_res[(int64_t)b * ldx + u] : 0.f;
  // the slices are read four at a time before any is added (sixteen loads in flight instead of a round trip
  // to memory per slice); the additions keep the order of the slices
  int p = 0;
  for (; p + 4 <= nparts; p += 4) {
    float v[4][4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const float* q = part + ((int64_t)(p + s) * B + b) * 4 * U;
      v[s][0] = q[u]; v[s][1] = q[U + u]; v[s][2] = q[2 * U + u]; v[s][3] = q[3 * U + u];
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) { gi += v[s][0]; gj += v[s][1]; gf += v[s][2]; go += v[s][3]; }
  }
  for (; p < nparts; ++p) {
    const float* q = part + ((int64_t)p * B + b) * 4 * U;
    gi += q[u]; gj += q[U + u]; gf += q[2 * U + u]; go += q[3 * U + u];
  }
  const float i = sigmoidf_(gi), j = tanhf(gj), f = sigmoidf_(gf + forget_bias), o = sigmoidf_(go);
  const float cn = cp * f + i * j;
  const float hn = tanhf(cn) * o;
  g[u] = i; g[U + u] = j; g[2 * U + u] = f; g[3 * U + u] = o;
  c[idx] = cn;
  h[(int64_t)b * ldh + u] = hn;
  if (y) y[(int64_t)b * ldy + u] = hn + xr;
}

// Backward of one step: dh = dy[t] + dh_rec, dc = dc_rec + dh*o*(1 - tanh(c)^2); writes the four
// pre-activation gate gradients, leaves dc*f in dc_rec for step t-1 and zeroes `clear` [B,U].
// The recurrent gradient comes as dh_rec [B,U] (nullable) and / or as part [nparts][B][U], the slices of dgates Wh^T.
__global__ __launch_bounds__(256) void lstm_cell_bwd_kernel(int B, int U, const float* __restrict__ gact,
                                                           const float* __restrict__ c, const float* __restrict__ c_prev,
                                                           const float* __restrict__ dy, int lddy,
                                                           const float* __restrict__ dh_rec, float* __restrict__ dc_rec,
                                                           int first, float* __restrict__ dgates,
                                                           const int32_t* __restrict__ len, int t, float* __restrict__ clear,
                                                           const float* __restrict__ part, int nparts) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= B * U) return;
  if (clear) clear[idx] = 0.f;  // the buffer the next recurrent product adds into
  const int b = idx / U, u = idx % U;
  if (len && t >= len[b]) {
    float* d = dgates + (int64_t)b * 4 * U;
    d[u] = 0.f; d[U + u] = 0.f; d[2 * U + u] = 0.f; d[3 * U + u] = 0.f;
    dc_rec[idx] = 0.f;
    return;
  }
  const float* g = gact + (int64_t)b * 4 * U;
  const float i = g[u], j = g[U + u], f = g[2 * U + u], o = g[3 * U + u];
  const float cv = c[idx];
  const float cp = c_prev ? c_prev[idx] : 0.f;
  const float dcr = first ? 0.f : dc_rec[idx];
  float dh = dy[(int64_t)b * lddy + u];
  if (!first) {
    if (dh_rec) dh += dh_rec[idx];
    // eight slices are read before any is added (one round trip to memory per eight instead of per slice);
    // the additions keep the order of the slices
    int p = 0;
    for (; p + 8 <= nparts; p += 8) {
      float v[8];
#pragma unroll
      for (int s = 0; s < 8; ++s) v[s] = part[((int64_t)(p + s) * B + b) * U + u];
#pragma unroll
      for (int s = 0; s < 8; ++s) dh += v[s];
    }
    for (; p < nparts; ++p) dh += part[((int64_t)p * B + b) * U + u];
  }
  const float tc = tanhf(cv);
  const float dc = dcr + dh * o * (1.f - tc * tc);
  float* d = dgates + (int64_t)b * 4 * U;
  d[u] = dc * j * i * (1.f - i);
  d[U + u] = dc * i * (1.f - j * j);
  d[2 * U + u] = dc * cp * f * (1.f - f);
  d[3 * U + u] = dh * tc * o * (1.f - o);
  dc_rec[idx] = dc * f;
}

// dst[t, b, :] = t < len[b] ? src[t, b, :] : 0 (the output past the end of a sequence is the constant 0)
__global__ __launch_bounds__(256) void mask_steps_kernel(int64_t total4, int B, int U4, const int32_t* __restrict__ len,
                                                        const f32x4* __restrict__ src, f32x4* __restrict__ dst) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total4; i += (int64_t)gridDim.x * 256) {
    const int64_t row = i / U4;
    const int t = (int)(row / B), b = (int)(row % B);
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
    dst[i] = t < len[b] ? src[i] : z;
  }
}

// fp32 GEMM helpers shared by the three stage kinds of this file
static int gnmt_gemm(hipStream_t stream, int am, int bm, int m, int n, int k, const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                     int64_t ldc, int flags, const float* bias, const void* residual) {
  ds_gemm_desc d;
  memset(&d, 0, sizeof(d));
  d.dtype = DS_F32; d.a_major = am; d.b_major = bm; d.m = m; d.n = n; d.k = k; d.lda = lda; d.ldb = ldb; d.ldc = ldc;
  d.batch = 1; d.batch_inner = 1; d.flags = flags; d.alpha = 1.f; d.a = a; d.b = b; d.c = c; d.bias = bias; d.residual = residual;
  return ds_gemm(&d, stream);
}
// reduction split of a product with few rows (the per-step recurrent products have only B of them)
static int gnmt_split_for(int m, int n, int k) {
  const int tiles = ((m + 63) / 64) * ((n + 63) / 64);
  int s = 256 / (tiles > 0 ? tiles : 1);
  const int ktiles = k / 32;
  if (s > ktiles / 4) s = ktiles / 4;
  return s < 1 ? 1 : s;
}
// c (fp32) += a[m,k] x b: the reduction is split across the chip and added with fp32 atomics
static int gnmt_gemm_accum_splitk(hipStream_t stream, int bm, int m, int n, int k, const void* a, int64_t lda, const void* b, int64_t ldb,
                                  float* c, int64_t ldc) {
  ds_gemm_desc d;
  memset(&d, 0, sizeof(d));
  d.dtype = DS_F32; d.a_major = DS_K_MAJOR; d.b_major = bm; d.m = m; d.n = n; d.k = k; d.lda = lda; d.ldb = ldb; d.ldc = ldc;
  d.batch = 1; d.batch_inner = 1; d.flags = DS_EPI_ACCUM; d.alpha = 1.f; d.a = a; d.b = b; d.c = c;
  return ds_gemm_splitk(&d, gnmt_split_for(m, n, k), stream);
}

// c[z] = a[:, z-th slice of k] x b[z-th slice of k, :]: the reduction of a product with few rows cut into `slices`
// independent products (a batched launch, plain stores) whose results the consumer adds up
static int gnmt_gemm_slices(hipStream_t stream, int bm, int m, int n, int k, int slices, const void* a, int64_t lda, const void* b,
                            int64_t ldb, float* parts) {
  ds_gemm_desc d;
  memset(&d, 0, sizeof(d));
  const int kc = k / slices;
  d.dtype = DS_F32; d.a_major = DS_K_MAJOR; d.b_major = bm; d.m = m; d.n = n; d.k = kc; d.lda = lda; d.ldb = ldb; d.ldc = n;
  d.batch = slices; d.batch_inner = slices;
  d.a_stride_inner = kc;
  d.b_stride_inner = bm == DS_K_MAJOR ? (int64_t)kc : (int64_t)kc * ldb;
  d.c_stride_inner = (int64_t)m * n;
  d.alpha = 1.f; d.a = a; d.b = b; d.c = parts;
  return ds_gemm(&d, stream);
}
// how many slices: enough 64x64 tiles for every CU, each slice a multiple of 32 (the fp32 k-tile) and at least 128 deep
static int gnmt_slices_for(int m, int n, int k) {
  const int tiles = ((m + 63) / 64) * ((n + 63) / 64);
  int s = 1;
  while (s < 32 && tiles * s < 256 && k % (2 * s * 32) == 0 && k / (2 * s) >= 128) s *= 2;
  return s;
}

struct Cell {
  int widx;        // kernel index in the weight list (bias = widx + 1)
  int n_in;        // input width
  bool reverse, residual;
  // byte offsets into a slot
  size_t x_off; int ldx;     // input activations [T*B, n_in]
  size_t h_off; int ldh;     // outputs h [T*B, U] (row stride ldh)
  size_t y_off;              // residual output y = h + x (residual cells only)
  size_t g_off, c_off;       // activated gates [T*B,4U], cell states [T*B,U]
};

struct GnmtStage : ds_stage {
  ds_gnmt_cfg gc;
  int B, T, U, L, R;  // R = T*B rows
  std::vector<Cell> cells;
  char* stash_base = nullptr;
  size_t slot_bytes = 0, ids_off = 0, len_off = 0, x0_off = 0, xb_off = 0;
  std::vector<char> slot_has_len;
  char* ws_base = nullptr;
  size_t ws_bytes = 0, ws_dg, ws_dx[2], ws_dc, ws_dym, ws_pf, ws_pb;
  int sl_f = 1, sl_b = 1;  // slices of the recurrent products h Wh (forward) and dgates Wh^T (backward)

  ~GnmtStage() override {
    if (stash_base) (void)hipFree(stash_base);
    if (ws_base) (void)hipFree(ws_base);
  }

  int init() {
    B = gc.batch; T = gc.seq; U = gc.units; L = gc.num_layers; R = B * T;
    const char* P = "dynamic_seq2seq/encoder/";
    char name[160];
    snprintf(name, sizeof(name), "%sembedding_encoder", P);
    winfo.push_back({name, gc.vocab, U});
    Arena sa;
    ids_off = sa.reserve((size_t)R * 4);
    len_off = sa.reserve((size_t)B * 4);
    x0_off = sa.reserve((size_t)R * U * 4);
    xb_off = sa.reserve((size_t)R * 2 * U * 4);
    size_t prev_out = 0;
    for (int i = 0; i < L + 1; ++i) {
      Cell c;
      memset(&c, 0, sizeof(c));
      const char* scope;
      char buf[96];
      if (i == 0) scope = "bidirectional_rnn/fw/basic_lstm_cell";
      else if (i == 1) scope = "bidirectional_rnn/bw/basic_lstm_cell";
      else { snprintf(buf, sizeof(buf), "rnn/multi_rnn_cell/cell_%d/rnn/basic_lstm_cell", i - 1); scope = buf; }
      c.n_in = (i == 2) ? 2 * U : U;
      c.reverse = (i == 1);
      c.residual = (i >= 3);
      c.widx = (int)winfo.size();
      snprintf(name, sizeof(name), "%s%s/kernel", P, scope);
      winfo.push_back({name, c.n_in + U, 4 * U});
      snprintf(name, sizeof(name), "%s%s/bias", P, scope);
      winfo.push_back({name, 1, 4 * U});
      c.g_off = sa.reserve((size_t)R * 4 * U * 4);
      c.c_off = sa.reserve((size_t)R * U * 4);
      if (i < 2) {
        c.x_off = x0_off; c.ldx = U;
        c.h_off = xb_off + (size_t)i * U * 4; c.ldh = 2 * U;
      } else if (i == 2) {
        c.x_off = xb_off; c.ldx = 2 * U;
        c.h_off = sa.reserve((size_t)R * U * 4); c.ldh = U;
        prev_out = c.h_off;
      } else {
        c.x_off = prev_out; c.ldx = U;
        c.h_off = sa.reserve((size_t)R * U * 4); c.ldh = U;
        c.y_off = sa.reserve((size_t)R * U * 4);
        prev_out = c.y_off;
      }
      cells.push_back(c);
    }
    slot_bytes = sa.used;
    DS_CHECK_HIP(hipMalloc((void**)&stash_base, slot_bytes * gc.stash_slots));
    slot_forwarded.assign(gc.stash_slots, 0);
    slot_has_len.assign(gc.stash_slots, 0);
    Arena wa;
    ws_dg = wa.reserve((size_t)R * 4 * U * 4);
    ws_dx[0] = wa.reserve((size_t)R * 2 * U * 4);
    ws_dx[1] = wa.reserve((size_t)R * 2 * U * 4);
    ws_dc = wa.reserve((size_t)B * U * 4);
    ws_dym = wa.reserve((size_t)R * U * 4);
    sl_f = gnmt_slices_for(B, 4 * U, U);
    sl_b = gnmt_slices_for(B, U, 4 * U);
    ws_pf = wa.reserve((size_t)sl_f * B * 4 * U * 4);  // forward's and backward's own: the two may run side by side
    ws_pb = wa.reserve((size_t)sl_b * B * U * 4);
    ws_bytes = wa.used;
    DS_CHECK_HIP(hipMalloc((void**)&ws_base, ws_bytes));
    return DS_OK;
  }

  size_t workspace_bytes() const override { return ws_bytes; }
  // forward touches its stash slot and its output only; the workspace is backward's
  bool overlap_safe() const override { return true; }
  size_t stash_bytes(int slots) const override { return slot_bytes * (size_t)slots; }
  int refresh_weights() override { return DS_OK; }  // fp32 kernels are used in place

  int gemm(int am, int bm, int m, int n, int k, const void* a, int64_t lda, const void* b, int64_t ldb, void* c, int64_t ldc,
           int flags, const float* bias, const void* residual) {
    return gnmt_gemm(stream, am, bm, m, n, k, a, lda, b, ldb, c, ldc, flags, bias, residual);
  }
  int gemm_accum_splitk(int bm, int m, int n, int k, const void* a, int64_t lda, const void* b, int64_t ldb, float* c, int64_t ldc) {
    return gnmt_gemm_accum_splitk(stream, bm, m, n, k, a, lda, b, ldb, c, ldc);
  }

  int set_lengths(int slot, const int32_t* lengths) {
    if (lengths)
      DS_CHECK_HIP(hipMemcpyAsync(stash_base + (size_t)slot * slot_bytes + len_off, lengths, (size_t)B * 4,
                                  hipMemcpyDeviceToDevice, stream));
    slot_has_len[slot] = lengths != nullptr;
    return DS_OK;
  }

  int forward(int slot, const void* in, const float*, void* out) override {
    ds_prio_scope prio(1);
    char* sp = stash_base + (size_t)slot * slot_bytes;
    const int32_t* len = slot_has_len[slot] ? (const int32_t*)(sp + len_off) : nullptr;
    DS_CHECK_HIP(hipMemcpyAsync(sp + ids_off, in, (size_t)R * 4, hipMemcpyDeviceToDevice, stream));
    hipLaunchKernelGGL(gnmt_embed_fwd_kernel, dim3((R + 3) / 4), dim3(256), 0, stream, B, T, U, gc.vocab,
                       (const int32_t*)(sp + ids_off), w[0], (float*)(sp + x0_off));
    DS_CHECK_LAUNCH();
    const int cell_grid = (B * U + 255) / 256;
    for (size_t ci = 0; ci < cells.size(); ++ci) {
      const Cell& c = cells[ci];
      const float* kernel = w[c.widx];
      const float* wh = kernel + (size_t)c.n_in * 4 * U;
      float* G = (float*)(sp + c.g_off);
      float* Cs = (float*)(sp + c.c_off);
      float* H = (float*)(sp + c.h_off);
      const float* X = (const float*)(sp + c.x_off);
      const bool last = ci + 1 == cells.size();
      float* Y = c.residual ? (last ? (float*)out : (float*)(sp + c.y_off)) : nullptr;
      // input half of the gates for every step: [T*B, n_in] x [n_in, 4U] + bias
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, R, 4 * U, c.n_in, X, c.ldx, kernel, 4 * U, G, 4 * U, DS_EPI_BIAS, w[c.widx + 1], nullptr));
      for (int s = 0; s < T; ++s) {
        const int t = c.reverse ? T - 1 - s : s;
        const int tp = c.reverse ? t + 1 : t - 1;  // the step whose state feeds this one
        float* g = G + (size_t)t * B * 4 * U;
        float* pf = (float*)(ws_base + ws_pf);
        if (s > 0)  // recurrent half h[tp] @ Wh in sl_f slices of the reduction; the cell kernel adds them to g
          DS_PROPAGATE(gnmt_gemm_slices(stream, DS_MN_MAJOR, B, 4 * U, U, sl_f, H + (size_t)tp * B * c.ldh, c.ldh, wh, 4 * U, pf));
        ds_prof_scope prof(stream, "lstm_cell_fwd_kernel", (double)B * U * 4 * (4 + 4 + 2 + (c.residual ? 2 : 1)), "B");
        hipLaunchKernelGGL(lstm_cell_fwd_kernel, dim3(cell_grid), dim3(256), 0, stream, B, U, gc.forget_bias, g,
                           s > 0 ? Cs + (size_t)tp * B * U : nullptr, Cs + (size_t)t * B * U, H + (size_t)t * B * c.ldh, c.ldh,
                           c.residual ? X + (size_t)t * B * c.ldx : nullptr, c.ldx, Y ? Y + (size_t)t * B * U : nullptr, U,
                           len, t, pf, s > 0 ? sl_f : 0);
        DS_CHECK_LAUNCH();
      }
      if (last && !c.residual)
        DS_CHECK_HIP(hipMemcpyAsync(out, H, (size_t)R * U * 4, hipMemcpyDeviceToDevice, stream));
    }
    return DS_OK;
  }

  int backward(int slot, const void* d_out, void*) override {
    ds_prio_scope prio(3);  // the chain every later pass waits on
    char* sp = stash_base + (size_t)slot * slot_bytes;
    float* dG = (float*)(ws_base + ws_dg);
    float* dc = (float*)(ws_base + ws_dc);
    const int cell_grid = (B * U + 255) / 256;
    const int32_t* len = slot_has_len[slot] ? (const int32_t*)(sp + len_off) : nullptr;
    const float* dY = (const float*)d_out;  // gradient w.r.t. the output of the cell being processed
    int lddy = U;
    if (len) {
      // the output past the end of a sequence is constant: no gradient enters there.  With that every gradient
      // tensor further down has zero rows at those steps by itself (zero gate gradients, masked residual).
      float* dym = (float*)(ws_base + ws_dym);
      const int64_t total4 = (int64_t)R * U / 4;
      hipLaunchKernelGGL(mask_steps_kernel, dim3((unsigned)((total4 + 255) / 256 > 4096 ? 4096 : (total4 + 255) / 256)), dim3(256), 0,
                         stream, total4, B, U / 4, len, (const f32x4*)d_out, (f32x4*)dym);
      DS_CHECK_LAUNCH();
      dY = dym;
    }
    int pp = 0;
    float* dXB = nullptr;  // gradient w.r.t. the fw|bw concatenation [R, 2U]
    float* dX0 = nullptr;
    for (int ci = (int)cells.size() - 1; ci >= 0; --ci) {
      const Cell& c = cells[ci];
      const float* kernel = w[c.widx];
      const float* wh = kernel + (size_t)c.n_in * 4 * U;
      const float* G = (const float*)(sp + c.g_off);
      const float* Cs = (const float*)(sp + c.c_off);
      const float* H = (const float*)(sp + c.h_off);
      const float* X = (const float*)(sp + c.x_off);
      if (ci < 2) { dY = dXB + (size_t)ci * U; lddy = 2 * U; }
      for (int s = T - 1; s >= 0; --s) {
        const int t = c.reverse ? T - 1 - s : s;
        const int tp = c.reverse ? t + 1 : t - 1;
        const int first = (s == T - 1);  // no recurrent gradient flows into the last step of the scan
        float* pb = (float*)(ws_base + ws_pb);  // slices of dgates Wh^T of the step scanned before this one
        {
          ds_prof_scope prof(stream, "lstm_cell_bwd_kernel", (double)B * U * 4 * (4 + 4 + 6), "B");
          hipLaunchKernelGGL(lstm_cell_bwd_kernel, dim3(cell_grid), dim3(256), 0, stream, B, U, G + (size_t)t * B * 4 * U,
                             Cs + (size_t)t * B * U, s > 0 ? Cs + (size_t)tp * B * U : nullptr, dY + (size_t)t * B * lddy, lddy,
                             (const float*)nullptr, dc, first, dG + (size_t)t * B * 4 * U, len, t, (float*)nullptr, pb, first ? 0 : sl_b);
          DS_CHECK_LAUNCH();
        }
        if (s > 0)  // dh for step tp: dgates[t] @ Wh^T, in sl_b slices the next cell kernel adds up
          DS_PROPAGATE(gnmt_gemm_slices(stream, DS_K_MAJOR, B, U, 4 * U, sl_b, dG + (size_t)t * B * 4 * U, 4 * U, wh, 4 * U, pb));
      }
      // parameter gradients over all steps
      DS_PROPAGATE(ds_colsum_accum(DS_F32, R, 4 * U, dG, 4 * U, g[c.widx + 1], stream));
      DS_PROPAGATE(gemm(DS_MN_MAJOR, DS_MN_MAJOR, c.n_in, 4 * U, R, X, c.ldx, dG, 4 * U, g[c.widx], 4 * U, DS_EPI_ACCUM, nullptr, nullptr));
      // dWh += Hprev^T dG: the state feeding step t is h[tp]; pair rows of H with the rows of dG one step later in scan order
      if (T > 1) {
        const float* Hp = c.reverse ? H + (size_t)B * c.ldh : H;
        const float* dGp = c.reverse ? dG : dG + (size_t)B * 4 * U;
        DS_PROPAGATE(gemm(DS_MN_MAJOR, DS_MN_MAJOR, U, 4 * U, (T - 1) * B, Hp, c.ldh, dGp, 4 * U, g[c.widx] + (size_t)c.n_in * 4 * U,
                          4 * U, DS_EPI_ACCUM, nullptr, nullptr));
      }
      // input gradient dX = dG @ Wx^T (+ dY through the residual connection)
      if (ci >= 2) {
        float* dX = (float*)(ws_base + ws_dx[pp]);
        DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, R, c.n_in, 4 * U, dG, 4 * U, kernel, 4 * U, dX, c.n_in,
                          c.residual ? DS_EPI_RESIDUAL : 0, nullptr, c.residual ? dY : nullptr));
        if (ci == 2) dXB = dX; else { dY = dX; lddy = U; }
        pp ^= 1;
      } else {
        // both directions read the embedding: dX0 = dG_bw Wx_bw^T, then += dG_fw Wx_fw^T
        if (ci == 1) dX0 = (float*)(ws_base + ws_dx[pp]);
        DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, R, U, 4 * U, dG, 4 * U, kernel, 4 * U, dX0, U, ci == 0 ? DS_EPI_RESIDUAL : 0,
                          nullptr, ci == 0 ? dX0 : nullptr));
      }
    }
    hipLaunchKernelGGL(gnmt_embed_bwd_kernel, dim3((R + 3) / 4), dim3(256), 0, stream, B, T, U, gc.vocab,
                       (const int32_t*)(sp + ids_off), dX0, g[0]);
    DS_CHECK_LAUNCH();
    return DS_OK;
  }
};

// The decoder cells of the second pipeline device, GNMTAttentionMultiCell_2 (gnmt_model.py:489-537) under
// dynamic_decode with a TrainingHelper (model.py:641-656): a scan over the padded target steps from the zero state.
// Cell l reads concat([cur_inp, attention]) - kernel rows [0,U) for the running input, [U,2U) for the attention,
// [2U,3U) for h - and, for l >= 2, adds the running input to its output (gnmt_residual_fn, :587-613).  The attention is
// a per-slot side input without gradient (the reference reads it from a non-trainable variable); a slot without one
// uses zeros and skips the products with the attention rows.
struct DecCell {
  int widx;
  bool residual;
  size_t g_off, c_off, h_off, y_off;
};

struct GnmtDecoderStage : ds_stage {
  ds_gnmt_cfg gc;
  int B, T, U, L, R;
  std::vector<DecCell> cells;
  char* stash_base = nullptr;
  size_t slot_bytes = 0, x0_off = 0, att_off = 0;
  std::vector<char> slot_has_att;
  char* ws_base = nullptr;
  size_t ws_bytes = 0, ws_dg, ws_dx[2], ws_dc, ws_pf, ws_pb;
  int sl_f = 1, sl_b = 1;  // slices of the recurrent products (see GnmtStage)

  ~GnmtDecoderStage() override {
    if (stash_base) (void)hipFree(stash_base);
    if (ws_base) (void)hipFree(ws_base);
  }

  int init() {
    B = gc.batch; T = gc.seq; U = gc.units; L = gc.num_layers; R = B * T;
    Arena sa;
    x0_off = sa.reserve((size_t)R * U * 4);
    att_off = sa.reserve((size_t)R * U * 4);
    char name[160];
    for (int i = 0; i < L; ++i) {
      const int layer = gc.first_layer + i;
      DecCell c;
      memset(&c, 0, sizeof(c));
      c.residual = layer >= 2;
      c.widx = (int)winfo.size();
      snprintf(name, sizeof(name), "dynamic_seq2seq/decoder/multi_rnn_cell_part2/cell_%d/basic_lstm_cell/kernel", layer);
      winfo.push_back({name, 3 * U, 4 * U});
      snprintf(name, sizeof(name), "dynamic_seq2seq/decoder/multi_rnn_cell_part2/cell_%d/basic_lstm_cell/bias", layer);
      winfo.push_back({name, 1, 4 * U});
      c.g_off = sa.reserve((size_t)R * 4 * U * 4);
      c.c_off = sa.reserve((size_t)R * U * 4);
      c.h_off = sa.reserve((size_t)R * U * 4);
      if (c.residual && i + 1 < L) c.y_off = sa.reserve((size_t)R * U * 4);
      cells.push_back(c);
    }
    slot_bytes = sa.used;
    DS_CHECK_HIP(hipMalloc((void**)&stash_base, slot_bytes * gc.stash_slots));
    slot_forwarded.assign(gc.stash_slots, 0);
    slot_has_att.assign(gc.stash_slots, 0);
    Arena wa;
    ws_dg = wa.reserve((size_t)R * 4 * U * 4);
    ws_dx[0] = wa.reserve((size_t)R * U * 4);
    ws_dx[1] = wa.reserve((size_t)R * U * 4);
    ws_dc = wa.reserve((size_t)B * U * 4);
    sl_f = gnmt_slices_for(B, 4 * U, U);
    sl_b = gnmt_slices_for(B, U, 4 * U);
    ws_pf = wa.reserve((size_t)sl_f * B * 4 * U * 4);
    ws_pb = wa.reserve((size_t)sl_b * B * U * 4);
    ws_bytes = wa.used;
    DS_CHECK_HIP(hipMalloc((void**)&ws_base, ws_bytes));
    return DS_OK;
  }

  size_t workspace_bytes() const override { return ws_bytes; }
  bool overlap_safe() const override { return true; }  // forward touches its stash slot and its output only
  size_t stash_bytes(int slots) const override { return slot_bytes * (size_t)slots; }
  int refresh_weights() override { return DS_OK; }

  int gemm(int am, int bm, int m, int n, int k, const void* a, int64_t lda, const void* b, int64_t ldb, void* c, int64_t ldc,
           int flags, const float* bias, const void* residual) {
    return gnmt_gemm(stream, am, bm, m, n, k, a, lda, b, ldb, c, ldc, flags, bias, residual);
  }
  int gemm_accum_splitk(int bm, int m, int n, int k, const void* a, int64_t lda, const void* b, int64_t ldb, float* c, int64_t ldc) {
    return gnmt_gemm_accum_splitk(stream, bm, m, n, k, a, lda, b, ldb, c, ldc);
  }

  int set_attention(int slot, const float* attention) {
    if (attention)
      DS_CHECK_HIP(hipMemcpyAsync(stash_base + (size_t)slot * slot_bytes + att_off, attention, (size_t)R * U * 4, hipMemcpyDeviceToDevice,
                                  stream));
    slot_has_att[slot] = attention != nullptr;
    return DS_OK;
  }

  int forward(int slot, const void* in, const float*, void* out) override {
    ds_prio_scope prio(1);
    char* sp = stash_base + (size_t)slot * slot_bytes;
    const float* att = slot_has_att[slot] ? (const float*)(sp + att_off) : nullptr;
    DS_CHECK_HIP(hipMemcpyAsync(sp + x0_off, in, (size_t)R * U * 4, hipMemcpyDeviceToDevice, stream));
    const int cell_grid = (B * U + 255) / 256;
    const float* X = (const float*)(sp + x0_off);
    for (size_t ci = 0; ci < cells.size(); ++ci) {
      const DecCell& c = cells[ci];
      const float* kernel = w[c.widx];
      const float* wa = kernel + (size_t)U * 4 * U;
      const float* wh = kernel + (size_t)2 * U * 4 * U;
      float* G = (float*)(sp + c.g_off);
      float* Cs = (float*)(sp + c.c_off);
      float* H = (float*)(sp + c.h_off);
      const bool last = ci + 1 == cells.size();
      float* Y = c.residual ? (last ? (float*)out : (float*)(sp + c.y_off)) : nullptr;
      // input part of the gates for every step: x Wx + bias (+ attention Wa)
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, R, 4 * U, U, X, U, kernel, 4 * U, G, 4 * U, DS_EPI_BIAS, w[c.widx + 1], nullptr));
      if (att) DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, R, 4 * U, U, att, U, wa, 4 * U, G, 4 * U, DS_EPI_ACCUM, nullptr, nullptr));
      for (int t = 0; t < T; ++t) {
        float* g = G + (size_t)t * B * 4 * U;
        float* pf = (float*)(ws_base + ws_pf);
        if (t > 0) DS_PROPAGATE(gnmt_gemm_slices(stream, DS_MN_MAJOR, B, 4 * U, U, sl_f, H + (size_t)(t - 1) * B * U, U, wh, 4 * U, pf));
        ds_prof_scope prof(stream, "lstm_cell_fwd_kernel", (double)B * U * 4 * (4 + 4 + 2 + (c.residual ? 2 : 1)), "B");
        hipLaunchKernelGGL(lstm_cell_fwd_kernel, dim3(cell_grid), dim3(256), 0, stream, B, U, gc.forget_bias, g,
                           t > 0 ? Cs + (size_t)(t - 1) * B * U : nullptr, Cs + (size_t)t * B * U, H + (size_t)t * B * U, U,
                           c.residual ? X + (size_t)t * B * U : nullptr, U, Y ? Y + (size_t)t * B * U : nullptr, U,
                           (const int32_t*)nullptr, t, pf, t > 0 ? sl_f : 0);
        DS_CHECK_LAUNCH();
      }
      if (last && !c.residual) DS_CHECK_HIP(hipMemcpyAsync(out, H, (size_t)R * U * 4, hipMemcpyDeviceToDevice, stream));
      X = c.residual ? Y : H;
    }
    return DS_OK;
  }

  int backward(int slot, const void* d_out, void* d_in) override {
    ds_prio_scope prio(3);
    char* sp = stash_base + (size_t)slot * slot_bytes;
    const float* att = slot_has_att[slot] ? (const float*)(sp + att_off) : nullptr;
    float* dG = (float*)(ws_base + ws_dg);
    float* dc = (float*)(ws_base + ws_dc);
    const int cell_grid = (B * U + 255) / 256;
    const float* dY = (const float*)d_out;
    int pp = 0;
    for (int ci = (int)cells.size() - 1; ci >= 0; --ci) {
      const DecCell& c = cells[ci];
      const float* kernel = w[c.widx];
      const float* wh = kernel + (size_t)2 * U * 4 * U;
      const float* G = (const float*)(sp + c.g_off);
      const float* Cs = (const float*)(sp + c.c_off);
      const float* H = (const float*)(sp + c.h_off);
      const float* X = (const float*)(sp + x0_off);
      if (ci > 0) X = (const float*)(sp + (cells[ci - 1].residual ? cells[ci - 1].y_off : cells[ci - 1].h_off));
      for (int t = T - 1; t >= 0; --t) {
        const int first = (t == T - 1);
        float* pb = (float*)(ws_base + ws_pb);
        {
          ds_prof_scope prof(stream, "lstm_cell_bwd_kernel", (double)B * U * 4 * (4 + 4 + 6), "B");
          hipLaunchKernelGGL(lstm_cell_bwd_kernel, dim3(cell_grid), dim3(256), 0, stream, B, U, G + (size_t)t * B * 4 * U,
                             Cs + (size_t)t * B * U, t > 0 ? Cs + (size_t)(t - 1) * B * U : nullptr, dY + (size_t)t * B * U, U,
                             (const float*)nullptr, dc, first, dG + (size_t)t * B * 4 * U, (const int32_t*)nullptr, t, (float*)nullptr, pb,
                             first ? 0 : sl_b);
          DS_CHECK_LAUNCH();
        }
        if (t > 0) DS_PROPAGATE(gnmt_gemm_slices(stream, DS_K_MAJOR, B, U, 4 * U, sl_b, dG + (size_t)t * B * 4 * U, 4 * U, wh, 4 * U, pb));
      }
      float* gk = g[c.widx];
      DS_PROPAGATE(ds_colsum_accum(DS_F32, R, 4 * U, dG, 4 * U, g[c.widx + 1], stream));
      DS_PROPAGATE(gemm(DS_MN_MAJOR, DS_MN_MAJOR, U, 4 * U, R, X, U, dG, 4 * U, gk, 4 * U, DS_EPI_ACCUM, nullptr, nullptr));
      if (att)
        DS_PROPAGATE(gemm(DS_MN_MAJOR, DS_MN_MAJOR, U, 4 * U, R, att, U, dG, 4 * U, gk + (size_t)U * 4 * U, 4 * U, DS_EPI_ACCUM, nullptr, nullptr));
      if (T > 1)
        DS_PROPAGATE(gemm(DS_MN_MAJOR, DS_MN_MAJOR, U, 4 * U, (T - 1) * B, H, U, dG + (size_t)B * 4 * U, 4 * U, gk + (size_t)2 * U * 4 * U,
                          4 * U, DS_EPI_ACCUM, nullptr, nullptr));
      // gradient of the running input: dG Wx^T (+ dY through the residual connection); none flows into the attention
      float* dX = ci > 0 ? (float*)(ws_base + ws_dx[pp]) : (float*)d_in;
      if (dX)
        DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, R, U, 4 * U, dG, 4 * U, kernel, 4 * U, dX, U, c.residual ? DS_EPI_RESIDUAL : 0, nullptr,
                          c.residual ? dY : nullptr));
      dY = dX;
      pp ^= 1;
    }
    return DS_OK;
  }
};

// ---------------------------------------------------------------------------------------------------------
// Decoder cell 0 under the attention wrapper: the first device's share of the decoder (gnmt_model.py:309-325,
// :366-374; model.py:622-640).  Per target step t:
//   gates = [emb_t | attention_{t-1} | h_{t-1}] K + bias -> (h_t, c_t);  pq = h_t W_q;
//   score[b, j] = sum_u nv[u] tanh(keys[b, j, u] + pq[b, u] + attention_b[u]) for j < source length, nv = g v / ||v||;
//   alignments = softmax_j;  attention_t = sum_j alignments[b, j] values[b, j, :]
// with values = the memory (encoder outputs) zeroed past each source length, keys = values W_mem.

// values[b, j, :] = j < len[b] ? memory[j, b, :] : 0 (batch-major); block 0 also forms nv = g v / ||v||
__global__ __launch_bounds__(256) void att_prep_kernel(int B, int S, int U, const float* __restrict__ memory, const int32_t* __restrict__ len,
                                                      float* __restrict__ values, const float* __restrict__ v, const float* __restrict__ gsc,
                                                      float* __restrict__ nv) {
  __shared__ float red[4];
  const int row = blockIdx.x;  // b * S + j
  const int b = row / S, j = row % S;
  const bool live = !len || j < len[b];
  for (int u = threadIdx.x; u < U; u += 256) values[(int64_t)row * U + u] = live ? memory[((int64_t)j * B + b) * U + u] : 0.f;
  if (row == 0) {
    float ss = 0.f;
    for (int u = threadIdx.x; u < U; u += 256) ss += v[u] * v[u];
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float sc = gsc[0] * rsqrtf(red[0] + red[1] + red[2] + red[3]);
    for (int u = threadIdx.x; u < U; u += 256) nv[u] = sc * v[u];
  }
}

constexpr int ATT_MAX_S = 512;

// One wave per (sample b, source step j): score[b][j] = sum_u nv[u] tanh(keys[b,j,u] + pq[b,u] + bias[u]) (raw, unmasked;
// steps past the source length are skipped: the next kernel never reads them)
__global__ __launch_bounds__(256) void att_score_kernel(int B, int S, int U, const float* __restrict__ keys, const float* __restrict__ pq,
                                                       const float* __restrict__ nv, const float* __restrict__ bias,
                                                       const int32_t* __restrict__ len, float* __restrict__ score) {
  const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= B * S) return;
  const int b = row / S, j = row % S;
  if (len && j >= len[b]) return;
  const float* k = keys + (int64_t)row * U;
  float a = 0.f;
  for (int u = lane * 4; u < U; u += 256) {
    const f32x4 kv = *reinterpret_cast<const f32x4*>(k + u);
    const f32x4 qv = *reinterpret_cast<const f32x4*>(pq + (int64_t)b * U + u);
    const f32x4 bv = *reinterpret_cast<const f32x4*>(bias + u);
    const f32x4 vv = *reinterpret_cast<const f32x4*>(nv + u);
#pragma unroll
    for (int e = 0; e < 4; ++e) a += vv[e] * tanhf(kv[e] + qv[e] + bv[e]);
  }
  a = wave_sum(a);
  if (lane == 0) score[row] = a;
}

// grid (ceil(U/256), B): softmax of sample b's raw scores over its valid source steps (every block of the sample repeats
// it: at most a few hundred values; the sample's first block writes the alignments, zero past the source length), then
// the context for the block's 256 units
__global__ __launch_bounds__(256) void att_context_kernel(int S, int U, const float* __restrict__ score, const float* __restrict__ values,
                                                         const int32_t* __restrict__ len, float* __restrict__ align,
                                                         float* __restrict__ ctx, int ldc) {
  __shared__ float sc[ATT_MAX_S];
  __shared__ float red[4];
  const int b = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int n = len ? len[b] : S;
  n = n < 0 ? 0 : (n > S ? S : n);
  float mx = -INFINITY;
  for (int j = threadIdx.x; j < n; j += 256) { sc[j] = score[(int64_t)b * S + j]; mx = fmaxf(mx, sc[j]); }
  mx = wave_max(mx);
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float sum = 0.f;
  for (int j = threadIdx.x; j < n; j += 256) sum += expf(sc[j] - mx);
  sum = wave_sum(sum);
  if (lane == 0) red[wave] = sum;
  __syncthreads();
  sum = red[0] + red[1] + red[2] + red[3];
  for (int j = threadIdx.x; j < S; j += 256) {
    const float p = j < n ? expf(sc[j] - mx) / sum : 0.f;
    if (j < n) sc[j] = p;
    if (blockIdx.x == 0) align[(int64_t)b * S + j] = p;
  }
  __syncthreads();
  const int u = blockIdx.x * 256 + threadIdx.x;
  if (u < U) {
    float c = 0.f;
    for (int j = 0; j < n; ++j) c += sc[j] * values[((int64_t)b * S + j) * U + u];
    ctx[(int64_t)b * ldc + u] = c;
  }
}

// One wave per (b, j): d alignment[b][j] = datt[b] . values[b, j]  (datt = d loss / d attention of this step)
__global__ __launch_bounds__(256) void att_dalign_kernel(int B, int S, int U, const float* __restrict__ values, const float* __restrict__ datt,
                                                        const int32_t* __restrict__ len, float* __restrict__ da) {
  const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= B * S) return;
  const int b = row / S, j = row % S;
  if (len && j >= len[b]) return;
  const float* vj = values + (int64_t)row * U;
  const float* d = datt + (int64_t)b * U;
  float a = 0.f;
  for (int u = lane * 4; u < U; u += 256) {
    const f32x4 x = *reinterpret_cast<const f32x4*>(vj + u);
    const f32x4 y = *reinterpret_cast<const f32x4*>(d + u);
    a += x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3];
  }
  a = wave_sum(a);
  if (lane == 0) da[row] = a;
}

// grid (ceil(U/256), B): the rest of one step's attention gradient for the block's 256 units of sample b.  datt [B,U] is
// consumed and cleared; dkeys / dvalues [B,S,U] are added to; dpq [B,U] is written; dnv / dbias [U] get atomic adds.
__global__ __launch_bounds__(256) void att_grad_kernel(int S, int U, const float* __restrict__ keys, const float* __restrict__ pq,
                                                      const float* __restrict__ nv, const float* __restrict__ bias,
                                                      const int32_t* __restrict__ len, const float* __restrict__ align,
                                                      const float* __restrict__ da, float* __restrict__ datt, float* __restrict__ dpq,
                                                      float* __restrict__ dkeys, float* __restrict__ dvalues, float* __restrict__ dnv,
                                                      float* __restrict__ dbias) {
  __shared__ float al[ATT_MAX_S];
  __shared__ float ds[ATT_MAX_S];
  __shared__ float red[4];
  const int b = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int n = len ? len[b] : S;
  n = n < 0 ? 0 : (n > S ? S : n);
  float s = 0.f;
  for (int j = threadIdx.x; j < n; j += 256) {
    al[j] = align[(int64_t)b * S + j];
    ds[j] = da[(int64_t)b * S + j];
    s += al[j] * ds[j];
  }
  s = wave_sum(s);
  if (lane == 0) red[wave] = s;
  __syncthreads();
  s = red[0] + red[1] + red[2] + red[3];
  for (int j = threadIdx.x; j < n; j += 256) ds[j] = al[j] * (ds[j] - s);  // d score[j]
  __syncthreads();
  const int u = blockIdx.x * 256 + threadIdx.x;
  if (u >= U) return;
  const float q = pq[(int64_t)b * U + u] + bias[u], v = nv[u], dat = datt[(int64_t)b * U + u];
  float acc_pq = 0.f, acc_nv = 0.f;
  for (int j = 0; j < n; ++j) {
    const int64_t o = ((int64_t)b * S + j) * U + u;
    const float th = tanhf(keys[o] + q);
    const float d = ds[j] * v * (1.f - th * th);
    dkeys[o] += d;
    dvalues[o] += al[j] * dat;
    acc_pq += d;
    acc_nv += ds[j] * th;
  }
  dpq[(int64_t)b * U + u] = acc_pq;
  atomicAdd(dbias + u, acc_pq);
  atomicAdd(dnv + u, acc_nv);
  datt[(int64_t)b * U + u] = 0.f;
}

// d memory[j, b, :] = j < len[b] ? dvalues[b, j, :] : 0
__global__ __launch_bounds__(256) void att_dmemory_kernel(int B, int S, int U, const float* __restrict__ dvalues, const int32_t* __restrict__ len,
                                                         float* __restrict__ dmem) {
  const int row = blockIdx.x, b = row / S, j = row % S;
  const bool live = !len || j < len[b];
  for (int u = threadIdx.x; u < U; u += 256) dmem[((int64_t)j * B + b) * U + u] = live ? dvalues[(int64_t)row * U + u] : 0.f;
}

// nv = g v / ||v||:  dg += dnv . v / ||v||;  dv += g / ||v|| (dnv - (dnv . v) v / ||v||^2)     (one block)
__global__ __launch_bounds__(256) void att_vg_bwd_kernel(int U, const float* __restrict__ dnv, const float* __restrict__ v,
                                                        const float* __restrict__ gsc, float* __restrict__ dv, float* __restrict__ dg) {
  __shared__ float r0[4], r1[4];
  float dot = 0.f, ss = 0.f;
  for (int u = threadIdx.x; u < U; u += 256) { dot += dnv[u] * v[u]; ss += v[u] * v[u]; }
  dot = wave_sum(dot); ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) { r0[threadIdx.x >> 6] = dot; r1[threadIdx.x >> 6] = ss; }
  __syncthreads();
  dot = r0[0] + r0[1] + r0[2] + r0[3];
  ss = r1[0] + r1[1] + r1[2] + r1[3];
  const float inv = rsqrtf(ss), g = gsc[0];
  for (int u = threadIdx.x; u < U; u += 256) dv[u] += g * inv * (dnv[u] - dot * v[u] / ss);
  if (threadIdx.x == 0) dg[0] += dot * inv;
}

__global__ __launch_bounds__(256) void gnmt_fill0_kernel(float* __restrict__ p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) p[i] = 0.f;
}

struct GnmtAttentionStage : ds_stage {
  ds_gnmt_cfg gc;
  int B, T, S, U, R, RS;
  enum { W_EMB, W_K, W_BIAS, W_MEM, W_Q, W_V, W_G, W_B };
  char* stash_base = nullptr;
  size_t slot_bytes = 0, ids_off, len_off, nv_off, val_off, key_off, emb_off, ah_off, g_off, c_off, al_off, pq_off, sc_off;
  std::vector<char> slot_has_len;
  std::vector<float*> slot_att_out;
  char* ws_base = nullptr;
  size_t ws_bytes = 0, ws_dg, ws_dah[2], ws_dc, ws_dpq, ws_dkeys, ws_dval, ws_dnv, ws_demb, ws_da;

  ~GnmtAttentionStage() override {
    if (stash_base) (void)hipFree(stash_base);
    if (ws_base) (void)hipFree(ws_base);
  }

  int init() {
    B = gc.batch; T = gc.seq; S = gc.src_seq; U = gc.units; R = B * T; RS = B * S;
    const char* P = "dynamic_seq2seq/decoder/";
    const char* A = "multi_rnn_cell_part1/cell_0_attention/attention/";
    char name[200];
    snprintf(name, sizeof(name), "%sembedding_decoder", P); winfo.push_back({name, gc.vocab, U});
    snprintf(name, sizeof(name), "%s%sbasic_lstm_cell/kernel", P, A); winfo.push_back({name, 3 * U, 4 * U});
    snprintf(name, sizeof(name), "%s%sbasic_lstm_cell/bias", P, A); winfo.push_back({name, 1, 4 * U});
    snprintf(name, sizeof(name), "%smemory_layer/kernel", P); winfo.push_back({name, U, U});
    snprintf(name, sizeof(name), "%s%sbahdanau_attention/query_layer/kernel", P, A); winfo.push_back({name, U, U});
    snprintf(name, sizeof(name), "%s%sbahdanau_attention/attention_v", P, A); winfo.push_back({name, 1, U});
    snprintf(name, sizeof(name), "%s%sbahdanau_attention/attention_g", P, A); winfo.push_back({name, 1, 1});
    snprintf(name, sizeof(name), "%s%sbahdanau_attention/attention_b", P, A); winfo.push_back({name, 1, U});
    Arena sa;
    ids_off = sa.reserve((size_t)R * 4);
    len_off = sa.reserve((size_t)B * 4);
    nv_off = sa.reserve((size_t)U * 4);
    val_off = sa.reserve((size_t)RS * U * 4);
    key_off = sa.reserve((size_t)RS * U * 4);
    emb_off = sa.reserve((size_t)R * U * 4);
    ah_off = sa.reserve((size_t)(T + 1) * B * 2 * U * 4);  // block t = [attention_{t-1} | h_{t-1}], block 0 zero
    g_off = sa.reserve((size_t)R * 4 * U * 4);
    c_off = sa.reserve((size_t)R * U * 4);
    al_off = sa.reserve((size_t)T * RS * 4);
    pq_off = sa.reserve((size_t)R * U * 4);
    sc_off = sa.reserve((size_t)RS * 4);   // raw scores of the step being computed
    slot_bytes = sa.used;
    DS_CHECK_HIP(hipMalloc((void**)&stash_base, slot_bytes * gc.stash_slots));
    slot_forwarded.assign(gc.stash_slots, 0);
    slot_has_len.assign(gc.stash_slots, 0);
    slot_att_out.assign(gc.stash_slots, nullptr);
    Arena wa;
    ws_dg = wa.reserve((size_t)R * 4 * U * 4);
    // gradient of [attention_{t-1} | h_{t-1}] as two [B, U] blocks, one product fills both; two of them in alternation
    ws_dah[0] = wa.reserve((size_t)2 * B * U * 4);
    ws_dah[1] = wa.reserve((size_t)2 * B * U * 4);
    ws_dc = wa.reserve((size_t)B * U * 4);
    ws_dpq = wa.reserve((size_t)R * U * 4);
    ws_dkeys = wa.reserve((size_t)RS * U * 4);
    ws_dval = wa.reserve((size_t)RS * U * 4);
    ws_dnv = wa.reserve((size_t)U * 4);
    ws_demb = wa.reserve((size_t)R * U * 4);
    ws_da = wa.reserve((size_t)RS * 4);
    ws_bytes = wa.used;
    DS_CHECK_HIP(hipMalloc((void**)&ws_base, ws_bytes));
    return DS_OK;
  }

  size_t workspace_bytes() const override { return ws_bytes; }
  bool overlap_safe() const override { return true; }  // forward touches its stash slot and its outputs only
  size_t stash_bytes(int slots) const override { return slot_bytes * (size_t)slots; }
  int refresh_weights() override { return DS_OK; }

  int gemm(int am, int bm, int m, int n, int k, const void* a, int64_t lda, const void* b, int64_t ldb, void* c, int64_t ldc,
           int flags, const float* bias, const void* residual) {
    return gnmt_gemm(stream, am, bm, m, n, k, a, lda, b, ldb, c, ldc, flags, bias, residual);
  }
  int gemm_accum_splitk(int bm, int m, int n, int k, const void* a, int64_t lda, const void* b, int64_t ldb, float* c, int64_t ldc) {
    return gnmt_gemm_accum_splitk(stream, bm, m, n, k, a, lda, b, ldb, c, ldc);
  }
  int fill0(float* p, int64_t n) {
    const int64_t blocks = (n + 255) / 256;
    hipLaunchKernelGGL(gnmt_fill0_kernel, dim3((unsigned)(blocks > 2048 ? 2048 : blocks)), dim3(256), 0, stream, p, n);
    DS_CHECK_LAUNCH();
    return DS_OK;
  }

  int set_inputs(int slot, const int32_t* target_input, const int32_t* source_lengths, float* attention_out) {
    char* sp = stash_base + (size_t)slot * slot_bytes;
    DS_CHECK_HIP(hipMemcpyAsync(sp + ids_off, target_input, (size_t)R * 4, hipMemcpyDeviceToDevice, stream));
    if (source_lengths) DS_CHECK_HIP(hipMemcpyAsync(sp + len_off, source_lengths, (size_t)B * 4, hipMemcpyDeviceToDevice, stream));
    slot_has_len[slot] = source_lengths != nullptr;
    slot_att_out[slot] = attention_out;
    return DS_OK;
  }

  int forward(int slot, const void* in, const float*, void* out) override {
    ds_prio_scope prio(1);
    char* sp = stash_base + (size_t)slot * slot_bytes;
    const int32_t* len = slot_has_len[slot] ? (const int32_t*)(sp + len_off) : nullptr;
    float* values = (float*)(sp + val_off);
    float* keys = (float*)(sp + key_off);
    float* nv = (float*)(sp + nv_off);
    float* emb = (float*)(sp + emb_off);
    float* AH = (float*)(sp + ah_off);
    float* G = (float*)(sp + g_off);
    float* Cs = (float*)(sp + c_off);
    float* AL = (float*)(sp + al_off);
    float* PQ = (float*)(sp + pq_off);
    const float* kernel = w[W_K];
    hipLaunchKernelGGL(att_prep_kernel, dim3(RS), dim3(256), 0, stream, B, S, U, (const float*)in, len, values, w[W_V], w[W_G], nv);
    hipLaunchKernelGGL(gnmt_embed_fwd_kernel, dim3((R + 3) / 4), dim3(256), 0, stream, B, T, U, gc.vocab, (const int32_t*)(sp + ids_off),
                       w[W_EMB], emb);
    DS_CHECK_LAUNCH();
    DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, RS, U, U, values, U, w[W_MEM], U, keys, U, 0, nullptr, nullptr));
    DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, R, 4 * U, U, emb, U, kernel, 4 * U, G, 4 * U, DS_EPI_BIAS, w[W_BIAS], nullptr));
    DS_PROPAGATE(fill0(AH, (int64_t)B * 2 * U));
    DS_PROPAGATE(fill0(PQ, (int64_t)R * U));
    const int cell_grid = (B * U + 255) / 256;
    for (int t = 0; t < T; ++t) {
      float* g = G + (size_t)t * B * 4 * U;
      float* ah = AH + (size_t)t * B * 2 * U;       // [attention_{t-1} | h_{t-1}]
      float* ah_next = ah + (size_t)B * 2 * U;
      if (t > 0) DS_PROPAGATE(gemm_accum_splitk(DS_MN_MAJOR, B, 4 * U, 2 * U, ah, 2 * U, kernel + (size_t)U * 4 * U, 4 * U, g, 4 * U));
      hipLaunchKernelGGL(lstm_cell_fwd_kernel, dim3(cell_grid), dim3(256), 0, stream, B, U, gc.forget_bias, g,
                         t > 0 ? Cs + (size_t)(t - 1) * B * U : nullptr, Cs + (size_t)t * B * U, ah_next + U, 2 * U, (const float*)nullptr, 0,
                         (float*)nullptr, 0, (const int32_t*)nullptr, t, (const float*)nullptr, 0);
      DS_CHECK_LAUNCH();
      float* pq = PQ + (size_t)t * B * U;
      DS_PROPAGATE(gemm_accum_splitk(DS_MN_MAJOR, B, U, U, ah_next + U, 2 * U, w[W_Q], U, pq, U));
      float* SC = (float*)(sp + sc_off);
      {
        ds_prof_scope prof(stream, "att_score_kernel", (double)RS * U * 4, "B");
        hipLaunchKernelGGL(att_score_kernel, dim3((RS + 3) / 4), dim3(256), 0, stream, B, S, U, keys, pq, nv, w[W_B], len, SC);
      }
      {
        ds_prof_scope prof(stream, "att_context_kernel", (double)RS * U * 4, "B");
        hipLaunchKernelGGL(att_context_kernel, dim3((U + 255) / 256, B), dim3(256), 0, stream, S, U, SC, values, len, AL + (size_t)t * RS,
                           ah_next, 2 * U);
      }
      DS_CHECK_LAUNCH();
    }
    // the cell outputs and, if asked for, the attention of every step, out of the [attention | h] blocks 1 .. T
    DS_CHECK_HIP(hipMemcpy2DAsync(out, (size_t)U * 4, AH + (size_t)B * 2 * U + U, (size_t)2 * U * 4, (size_t)U * 4, R, hipMemcpyDeviceToDevice,
                                  stream));
    if (slot_att_out[slot])
      DS_CHECK_HIP(hipMemcpy2DAsync(slot_att_out[slot], (size_t)U * 4, AH + (size_t)B * 2 * U, (size_t)2 * U * 4, (size_t)U * 4, R,
                                    hipMemcpyDeviceToDevice, stream));
    return DS_OK;
  }

  int backward(int slot, const void* d_out, void* d_in) override {
    ds_prio_scope prio(3);
    char* sp = stash_base + (size_t)slot * slot_bytes;
    const int32_t* len = slot_has_len[slot] ? (const int32_t*)(sp + len_off) : nullptr;
    const float* values = (const float*)(sp + val_off);
    const float* keys = (const float*)(sp + key_off);
    const float* nv = (const float*)(sp + nv_off);
    const float* emb = (const float*)(sp + emb_off);
    const float* AH = (const float*)(sp + ah_off);
    const float* G = (const float*)(sp + g_off);
    const float* Cs = (const float*)(sp + c_off);
    const float* AL = (const float*)(sp + al_off);
    const float* PQ = (const float*)(sp + pq_off);
    const float* kernel = w[W_K];
    float* dG = (float*)(ws_base + ws_dg);
    float* dc = (float*)(ws_base + ws_dc);
    float* dPQ = (float*)(ws_base + ws_dpq);
    float* dkeys = (float*)(ws_base + ws_dkeys);
    float* dval = (float*)(ws_base + ws_dval);
    float* dnv = (float*)(ws_base + ws_dnv);
    const float* dY = (const float*)d_out;
    // dah .. dnv are adjacent: the state gradients, the last step's dpq, the two [B,S,U] accumulators and dnv start at zero
    DS_PROPAGATE(fill0((float*)(ws_base + ws_dah[0]), (int64_t)((ws_demb - ws_dah[0]) / 4)));
    const int cell_grid = (B * U + 255) / 256;
    for (int t = T - 1; t >= 0; --t) {
      const int first = (t == T - 1);  // nothing downstream reads the last step's state or attention
      // block (t & 1): [d attention_t | d h_t] from step t + 1; the other block receives this step's
      float* datt = (float*)(ws_base + ws_dah[t & 1]);
      float* dh_in = datt + (size_t)B * U;
      float* datt_out = (float*)(ws_base + ws_dah[(t & 1) ^ 1]);
      float* dh_out = datt_out + (size_t)B * U;
      float* dpq = dPQ + (size_t)t * B * U;
      if (!first) {
        float* da = (float*)(ws_base + ws_da);
        {
          ds_prof_scope prof(stream, "att_dalign_kernel", (double)RS * U * 4, "B");
          hipLaunchKernelGGL(att_dalign_kernel, dim3((RS + 3) / 4), dim3(256), 0, stream, B, S, U, values, datt, len, da);
        }
        {
          ds_prof_scope prof(stream, "att_grad_kernel", (double)RS * U * 4 * 5, "B");
          hipLaunchKernelGGL(att_grad_kernel, dim3((U + 255) / 256, B), dim3(256), 0, stream, S, U, keys, PQ + (size_t)t * B * U, nv, w[W_B],
                             len, AL + (size_t)t * RS, da, datt, dpq, dkeys, dval, dnv, g[W_B]);
        }
        DS_CHECK_LAUNCH();
        // the query is the cell output: dh_t += dpq W_q^T
        DS_PROPAGATE(gemm_accum_splitk(DS_K_MAJOR, B, U, U, dpq, U, w[W_Q], U, dh_in, U));
      }
      hipLaunchKernelGGL(lstm_cell_bwd_kernel, dim3(cell_grid), dim3(256), 0, stream, B, U, G + (size_t)t * B * 4 * U, Cs + (size_t)t * B * U,
                         t > 0 ? Cs + (size_t)(t - 1) * B * U : nullptr, dY + (size_t)t * B * U, U, dh_in, dc, first, dG + (size_t)t * B * 4 * U,
                         (const int32_t*)nullptr, t, t > 0 ? dh_out : nullptr, (const float*)nullptr, 0);
      DS_CHECK_LAUNCH();
      if (t > 0) {
        // [d attention_{t-1} ; d h_{t-1}] = dgates_t x (attention rows ; h rows of the kernel)^T: one batched product.
        // Both targets are zero here: dh_out by the cell kernel above, datt_out by the att_grad_kernel that last read it.
        ds_gemm_desc d;
        memset(&d, 0, sizeof(d));
        d.dtype = DS_F32; d.a_major = DS_K_MAJOR; d.b_major = DS_K_MAJOR; d.m = B; d.n = U; d.k = 4 * U; d.lda = 4 * U; d.ldb = 4 * U; d.ldc = U;
        d.batch = 2; d.batch_inner = 2; d.b_stride_inner = (int64_t)U * 4 * U; d.c_stride_inner = (int64_t)B * U;
        d.flags = DS_EPI_ACCUM; d.alpha = 1.f; d.a = dG + (size_t)t * B * 4 * U; d.b = kernel + (size_t)U * 4 * U; d.c = datt_out;
        DS_PROPAGATE(ds_gemm_splitk(&d, gnmt_split_for(B, 2 * U, 4 * U), stream));
      }
    }
    // parameter gradients over all steps
    DS_PROPAGATE(ds_colsum_accum(DS_F32, R, 4 * U, dG, 4 * U, g[W_BIAS], stream));
    DS_PROPAGATE(gemm(DS_MN_MAJOR, DS_MN_MAJOR, U, 4 * U, R, emb, U, dG, 4 * U, g[W_K], 4 * U, DS_EPI_ACCUM, nullptr, nullptr));
    DS_PROPAGATE(gemm(DS_MN_MAJOR, DS_MN_MAJOR, 2 * U, 4 * U, R, AH, 2 * U, dG, 4 * U, g[W_K] + (size_t)U * 4 * U, 4 * U, DS_EPI_ACCUM, nullptr,
                      nullptr));
    DS_PROPAGATE(gemm(DS_MN_MAJOR, DS_MN_MAJOR, U, U, R, AH + (size_t)B * 2 * U + U, 2 * U, dPQ, U, g[W_Q], U, DS_EPI_ACCUM, nullptr, nullptr));
    DS_PROPAGATE(gemm(DS_MN_MAJOR, DS_MN_MAJOR, U, U, RS, values, U, dkeys, U, g[W_MEM], U, DS_EPI_ACCUM, nullptr, nullptr));
    hipLaunchKernelGGL(att_vg_bwd_kernel, dim3(1), dim3(256), 0, stream, U, dnv, w[W_V], w[W_G], g[W_V], g[W_G]);
    DS_CHECK_LAUNCH();
    // embedding rows
    float* demb = (float*)(ws_base + ws_demb);
    DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, R, U, 4 * U, dG, 4 * U, kernel, 4 * U, demb, U, 0, nullptr, nullptr));
    hipLaunchKernelGGL(gnmt_embed_bwd_kernel, dim3((R + 3) / 4), dim3(256), 0, stream, B, T, U, gc.vocab, (const int32_t*)(sp + ids_off), demb,
                       g[W_EMB]);
    DS_CHECK_LAUNCH();
    // the memory: through the values directly and through the keys
    if (d_in) {
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, RS, U, U, dkeys, U, w[W_MEM], U, dval, U, DS_EPI_RESIDUAL, nullptr, dval));
      hipLaunchKernelGGL(att_dmemory_kernel, dim3(RS), dim3(256), 0, stream, B, S, U, dval, len, (float*)d_in);
      DS_CHECK_LAUNCH();
    }
    return DS_OK;
  }
};

}  // namespace

extern "C" int ds_gnmt_stage_create(const ds_gnmt_cfg* c, void* stream, ds_stage** out) {
  DS_CHECK_ARG(c != nullptr && out != nullptr, "ds_gnmt_stage_create: null argument");
  *out = nullptr;
  DS_CHECK_ARG(c->dtype == DS_F32, "ds_gnmt_stage_create: only fp32 is built (dtype %d)", c->dtype);
  if (c->part == DS_GNMT_ATTENTION_CELL) {
    DS_CHECK_ARG(c->units > 0 && c->units % 4 == 0, "ds_gnmt_stage_create: num_units (%d) must be a positive multiple of 4", c->units);
    DS_CHECK_ARG(c->batch > 0 && c->seq > 0 && c->batch % 4 == 0 && c->vocab > 0,
                 "ds_gnmt_stage_create: batch (%d) must be a positive multiple of 4, seq (%d) and vocab (%d) positive", c->batch, c->seq, c->vocab);
    DS_CHECK_ARG(c->src_seq >= 1 && c->src_seq <= ATT_MAX_S, "ds_gnmt_stage_create: src_seq (%d) must be in [1, %d]", c->src_seq, ATT_MAX_S);
    DS_CHECK_ARG(c->stash_slots >= 1, "ds_gnmt_stage_create: stash_slots must be >= 1");
    GnmtAttentionStage* s = new GnmtAttentionStage();
    memset(&s->cfg, 0, sizeof(s->cfg));
    s->cfg.kind = DS_STAGE_GNMT;
    s->cfg.dtype = c->dtype;
    s->cfg.stash_slots = c->stash_slots;
    s->gc = *c;
    s->stream = (hipStream_t)stream;
    const int rc = s->init();
    if (rc != DS_OK) { delete s; return rc; }
    *out = s;
    return DS_OK;
  }
  DS_CHECK_ARG(c->part == DS_GNMT_ENCODER || c->part == DS_GNMT_DECODER_PART2, "ds_gnmt_stage_create: unknown part %d", c->part);
  if (c->part == DS_GNMT_DECODER_PART2) {
    DS_CHECK_ARG(c->num_layers >= 1 && c->first_layer >= 1, "ds_gnmt_stage_create: decoder part 2 holds cells first_layer >= 1 .. (got %d layers from %d)",
                 c->num_layers, c->first_layer);
    DS_CHECK_ARG(c->units > 0 && c->units % 4 == 0, "ds_gnmt_stage_create: num_units (%d) must be a positive multiple of 4", c->units);
    DS_CHECK_ARG(c->batch > 0 && c->seq > 0 && c->batch % 4 == 0, "ds_gnmt_stage_create: batch (%d) must be a positive multiple of 4, seq (%d) positive",
                 c->batch, c->seq);
    DS_CHECK_ARG(c->stash_slots >= 1, "ds_gnmt_stage_create: stash_slots must be >= 1");
    GnmtDecoderStage* s = new GnmtDecoderStage();
    memset(&s->cfg, 0, sizeof(s->cfg));
    s->cfg.kind = DS_STAGE_GNMT;
    s->cfg.dtype = c->dtype;
    s->cfg.stash_slots = c->stash_slots;
    s->gc = *c;
    s->stream = (hipStream_t)stream;
    const int rc = s->init();
    if (rc != DS_OK) { delete s; return rc; }
    *out = s;
    return DS_OK;
  }
  DS_CHECK_ARG(c->num_layers >= 2, "ds_gnmt_stage_create: the GNMT encoder has a bidirectional layer and at least one uni-directional layer");
  DS_CHECK_ARG(c->units > 0 && c->units % 4 == 0, "ds_gnmt_stage_create: num_units (%d) must be a positive multiple of 4", c->units);
  DS_CHECK_ARG(c->batch > 0 && c->seq > 0 && c->vocab > 0, "ds_gnmt_stage_create: non-positive shape");
  DS_CHECK_ARG(c->batch % 4 == 0, "ds_gnmt_stage_create: batch (%d) must be a multiple of 4", c->batch);
  DS_CHECK_ARG(c->stash_slots >= 1, "ds_gnmt_stage_create: stash_slots must be >= 1");
  GnmtStage* s = new GnmtStage();
  memset(&s->cfg, 0, sizeof(s->cfg));
  s->cfg.kind = DS_STAGE_GNMT;
  s->cfg.dtype = c->dtype;
  s->cfg.stash_slots = c->stash_slots;
  s->gc = *c;
  s->stream = (hipStream_t)stream;
  const int rc = s->init();
  if (rc != DS_OK) { delete s; return rc; }
  *out = s;
  return DS_OK;
}

extern "C" int ds_gnmt_stage_set_lengths(ds_stage* h, int slot, const int32_t* lengths) {
  DS_CHECK_ARG(h != nullptr, "ds_gnmt_stage_set_lengths: null handle");
  DS_CHECK_ARG(h->cfg.kind == DS_STAGE_GNMT, "ds_gnmt_stage_set_lengths: not a GNMT stage");
  DS_CHECK_ARG(slot >= 0 && slot < h->cfg.stash_slots, "ds_gnmt_stage_set_lengths: slot %d out of range", slot);
  GnmtStage* enc = dynamic_cast<GnmtStage*>(h);
  DS_CHECK_ARG(enc != nullptr, "ds_gnmt_stage_set_lengths: the decoder cells run every padded step (dynamic_decode without impute_finished)");
  DS_PROPAGATE(ds_stage_acquire_slot(h, slot));
  return enc->set_lengths(slot, lengths);
}

extern "C" int ds_gnmt_stage_set_attention(ds_stage* h, int slot, const float* attention) {
  DS_CHECK_ARG(h != nullptr, "ds_gnmt_stage_set_attention: null handle");
  GnmtDecoderStage* dec = h->cfg.kind == DS_STAGE_GNMT ? dynamic_cast<GnmtDecoderStage*>(h) : nullptr;
  DS_CHECK_ARG(dec != nullptr, "ds_gnmt_stage_set_attention: not a GNMT decoder stage");
  DS_CHECK_ARG(slot >= 0 && slot < h->cfg.stash_slots, "ds_gnmt_stage_set_attention: slot %d out of range", slot);
  DS_PROPAGATE(ds_stage_acquire_slot(h, slot));
  return dec->set_attention(slot, attention);
}

extern "C" int ds_gnmt_stage_set_decoder_inputs(ds_stage* h, int slot, const int32_t* target_input, const int32_t* source_sequence_length,
                                                float* attention_out) {
  DS_CHECK_ARG(h != nullptr, "ds_gnmt_stage_set_decoder_inputs: null handle");
  GnmtAttentionStage* st = h->cfg.kind == DS_STAGE_GNMT ? dynamic_cast<GnmtAttentionStage*>(h) : nullptr;
  DS_CHECK_ARG(st != nullptr, "ds_gnmt_stage_set_decoder_inputs: not a GNMT attention-cell stage");
  DS_CHECK_ARG(slot >= 0 && slot < h->cfg.stash_slots, "ds_gnmt_stage_set_decoder_inputs: slot %d out of range", slot);
  DS_CHECK_ARG(target_input != nullptr, "ds_gnmt_stage_set_decoder_inputs: null target_input");
  DS_PROPAGATE(ds_stage_acquire_slot(h, slot));
  return st->set_inputs(slot, target_input, source_sequence_length, attention_out);
}

// ------------------------------------------------------------------ the cell kernels on their own
extern "C" int ds_lstm_cell_fwd(int batch, int units, float forget_bias, float* gates, const float* c_prev, float* c, float* h,
                                const float* x_residual, float* y, void* stream) {
  DS_CHECK_ARG(batch > 0 && units > 0 && (int64_t)batch * units < ((int64_t)1 << 31), "ds_lstm_cell_fwd: bad shape (%d, %d)", batch, units);
  DS_CHECK_ARG(gates && c && h, "ds_lstm_cell_fwd: null pointer");
  DS_CHECK_ARG((x_residual == nullptr) == (y == nullptr), "ds_lstm_cell_fwd: x_residual and y come together (ResidualWrapper)");
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, "lstm_cell_fwd_kernel", (double)batch * units * 4 * (4 + 4 + 2 + (y ? 2 : 1)), "B");
  hipLaunchKernelGGL(lstm_cell_fwd_kernel, dim3((batch * units + 255) / 256), dim3(256), 0, s, batch, units, forget_bias, gates, c_prev, c, h,
                     units, x_residual, units, y, units, (const int32_t*)nullptr, 0, (const float*)nullptr, 0);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_lstm_cell_bwd(int batch, int units, const float* gates_act, const float* c, const float* c_prev, const float* dh,
                                float* dc, int first, float* dgates, void* stream) {
  DS_CHECK_ARG(batch > 0 && units > 0 && (int64_t)batch * units < ((int64_t)1 << 31), "ds_lstm_cell_bwd: bad shape (%d, %d)", batch, units);
  DS_CHECK_ARG(gates_act && c && dh && dc && dgates, "ds_lstm_cell_bwd: null pointer");
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, "lstm_cell_bwd_kernel", (double)batch * units * 4 * (4 + 4 + 6), "B");
  hipLaunchKernelGGL(lstm_cell_bwd_kernel, dim3((batch * units + 255) / 256), dim3(256), 0, s, batch, units, gates_act, c, c_prev, dh, units,
                     (const float*)nullptr, dc, first, dgates, (const int32_t*)nullptr, 0, (float*)nullptr, (const float*)nullptr, 0);
  DS_CHECK_LAUNCH();
  return DS_OK;
}
