// Error plumbing and build probe of the C ABI.
#include "common.h"

static thread_local char g_err[512] = "";

void ds_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char* ds_last_error(void) { return g_err; }
extern "C" const char* ds_build_target(void) { return "gfx950"; }

// ---------------------------------------------------------------- stage handle dispatch
#include <string.h>

#include "stage.h"

extern "C" int ds_stage_create(const ds_stage_cfg* cfg, void* stream, ds_stage** out) {
  DS_CHECK_ARG(cfg != nullptr && out != nullptr, "ds_stage_create: null argument");
  *out = nullptr;
  switch (cfg->kind) {
    case DS_STAGE_BERT: return ds_bert_stage_create(cfg, (hipStream_t)stream, out);
    default: ds_set_error("ds_stage_create: unknown stage kind %d", cfg->kind); return DS_EINVAL;
  }
}

extern "C" int ds_stage_destroy(ds_stage* h) {
  if (!h) return DS_OK;
  (void)hipStreamSynchronize(h->stream);
  delete h;
  return DS_OK;
}

extern "C" int ds_stage_num_weights(const ds_stage* h) { return h ? (int)h->winfo.size() : 0; }

extern "C" int ds_stage_weight_info(const ds_stage* h, int i, char* name_buf, size_t name_cap, int64_t* numel,
                                    int64_t* rows, int64_t* cols) {
  DS_CHECK_ARG(h != nullptr, "ds_stage_weight_info: null handle");
  DS_CHECK_ARG(i >= 0 && i < (int)h->winfo.size(), "ds_stage_weight_info: index %d out of range", i);
  const WeightInfo& w = h->winfo[i];
  if (name_buf && name_cap) {
    strncpy(name_buf, w.name.c_str(), name_cap - 1);
    name_buf[name_cap - 1] = 0;
  }
  if (numel) *numel = w.numel();
  if (rows) *rows = w.rows;
  if (cols) *cols = w.cols;
  return DS_OK;
}

extern "C" int ds_stage_bind_weights(ds_stage* h, int n, const void* const* weights, void* const* master_grads) {
  DS_CHECK_ARG(h != nullptr && weights != nullptr && master_grads != nullptr, "ds_stage_bind_weights: null argument");
  DS_CHECK_ARG(n == (int)h->winfo.size(), "ds_stage_bind_weights: got %d tensors, stage has %d", n, (int)h->winfo.size());
  for (int i = 0; i < n; ++i) {
    DS_CHECK_ARG(weights[i] && master_grads[i], "ds_stage_bind_weights: tensor %d (%s) is null", i, h->winfo[i].name.c_str());
    DS_CHECK_ARG(ds_aligned16(weights[i]) && ds_aligned16(master_grads[i]),
                 "ds_stage_bind_weights: tensor %d (%s) is not 16-byte aligned", i, h->winfo[i].name.c_str());
  }
  h->w.assign(n, nullptr);
  h->g.assign(n, nullptr);
  for (int i = 0; i < n; ++i) {
    h->w[i] = (const float*)weights[i];
    h->g[i] = (float*)master_grads[i];
  }
  h->bound = true;
  return h->refresh_weights();
}

extern "C" int ds_stage_refresh_weights(ds_stage* h) {
  DS_CHECK_ARG(h != nullptr, "ds_stage_refresh_weights: null handle");
  if (!h->bound) { ds_set_error("ds_stage_refresh_weights: weights not bound"); return DS_ESTATE; }
  return h->refresh_weights();
}

extern "C" int ds_stage_forward(ds_stage* h, int slot, const void* in, const float* key_mask, void* out) {
  DS_CHECK_ARG(h != nullptr && in != nullptr && out != nullptr, "ds_stage_forward: null argument");
  DS_CHECK_ARG(slot >= 0 && slot < h->cfg.stash_slots, "ds_stage_forward: slot %d out of range [0,%d)", slot, h->cfg.stash_slots);
  if (!h->bound) { ds_set_error("ds_stage_forward: weights not bound"); return DS_ESTATE; }
  if (h->slot_forwarded[slot]) {
    ds_set_error("ds_stage_forward: slot %d still holds a micro-batch whose backward has not run", slot);
    return DS_ESTATE;
  }
  DS_CHECK_ARG(ds_aligned16(in) && ds_aligned16(out), "ds_stage_forward: in/out must be 16-byte aligned");
  const int rc = h->forward(slot, in, key_mask, out);
  if (rc == DS_OK) h->slot_forwarded[slot] = 1;
  return rc;
}

extern "C" int ds_stage_backward(ds_stage* h, int slot, const void* d_out, void* d_in) {
  DS_CHECK_ARG(h != nullptr && d_out != nullptr, "ds_stage_backward: null argument");
  DS_CHECK_ARG(slot >= 0 && slot < h->cfg.stash_slots, "ds_stage_backward: slot %d out of range [0,%d)", slot, h->cfg.stash_slots);
  if (!h->slot_forwarded[slot]) {
    ds_set_error("ds_stage_backward: slot %d holds no forwarded micro-batch", slot);
    return DS_ESTATE;
  }
  DS_CHECK_ARG(ds_aligned16(d_out) && ds_aligned16(d_in), "ds_stage_backward: d_out/d_in must be 16-byte aligned");
  const int rc = h->backward(slot, d_out, d_in);
  h->slot_forwarded[slot] = 0;
  return rc;
}

extern "C" size_t ds_stage_workspace_bytes(const ds_stage* h) { return h ? h->workspace_bytes() : 0; }
extern "C" size_t ds_stage_stash_bytes(const ds_stage* h, int slots) { return h ? h->stash_bytes(slots) : 0; }

extern "C" int ds_stage_sync(ds_stage* h) {
  DS_CHECK_ARG(h != nullptr, "ds_stage_sync: null handle");
  DS_CHECK_HIP(hipStreamSynchronize(h->stream));
  return DS_OK;
}
