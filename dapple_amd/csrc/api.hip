// Error plumbing and build probe of the C ABI.
#include "common.h"

static thread_local char g_err[512] = "";

void ds_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// ---------------------------------------------------------------- per-launch timing
#include <map>
#include <string>
#include <vector>

namespace {
struct ProfEntry { std::string tag; const char* unit; double work; hipEvent_t a, b; };
bool g_prof_on = false;
std::vector<ProfEntry> g_prof;
std::vector<hipEvent_t> g_event_pool;
hipEvent_t take_event() {
  if (!g_event_pool.empty()) { hipEvent_t e = g_event_pool.back(); g_event_pool.pop_back(); return e; }
  hipEvent_t e = nullptr;
  (void)hipEventCreate(&e);
  return e;
}
}  // namespace

ds_prof_scope::ds_prof_scope(hipStream_t s, const char* tag, double work, const char* unit) : on(g_prof_on), stream(s) {
  if (!on) return;
  ProfEntry e{tag, unit, work, take_event(), take_event()};
  (void)hipEventRecord(e.a, s);
  g_prof.push_back(e);
}
ds_prof_scope::~ds_prof_scope() {
  if (on) (void)hipEventRecord(g_prof.back().b, stream);
}

extern "C" int ds_profile_enable(int on) {
  g_prof_on = on != 0;
  return DS_OK;
}

// Writes one line per kernel tag: "tag<TAB>launches<TAB>total_ms<TAB>total_work<TAB>unit\n" and clears the log.
extern "C" int ds_profile_dump(char* buf, size_t cap) {
  DS_CHECK_ARG(buf != nullptr && cap > 0, "ds_profile_dump: null buffer");
  struct Agg { long n = 0; double ms = 0, work = 0; const char* unit = ""; };
  std::map<std::string, Agg> agg;
  for (ProfEntry& e : g_prof) {
    DS_CHECK_HIP(hipEventSynchronize(e.b));
    float ms = 0.f;
    DS_CHECK_HIP(hipEventElapsedTime(&ms, e.a, e.b));
    Agg& a = agg[e.tag];
    a.n++; a.ms += ms; a.work += e.work; a.unit = e.unit;
    g_event_pool.push_back(e.a);
    g_event_pool.push_back(e.b);
  }
  g_prof.clear();
  size_t off = 0;
  buf[0] = 0;
  for (auto& kv : agg) {
    const int w = snprintf(buf + off, cap - off, "%s\t%ld\t%.6f\t%.6e\t%s\n", kv.first.c_str(), kv.second.n, kv.second.ms,
                           kv.second.work, kv.second.unit);
    if (w < 0 || (size_t)w >= cap - off) { ds_set_error("ds_profile_dump: buffer too small"); return DS_EINVAL; }
    off += w;
  }
  return DS_OK;
}

thread_local int ds_launch_prio = 0;

extern "C" const char* ds_last_error(void) { return g_err; }
extern "C" const char* ds_build_target(void) { return "gfx950"; }

// ---------------------------------------------------------------- stage handle dispatch
#include <stdlib.h>
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
  if (h->bwd_owned) {
    (void)hipStreamSynchronize(h->bwd_owned);
    (void)hipStreamSynchronize(h->wgrad_owned);
    for (hipEvent_t e : h->ev_forwarded) (void)hipEventDestroy(e);
    for (hipEvent_t e : h->ev_released) (void)hipEventDestroy(e);
    if (h->ev_join) (void)hipEventDestroy(h->ev_join);
    if (h->ev_dout) (void)hipEventDestroy(h->ev_dout);
    if (h->ev_pair) (void)hipEventDestroy(h->ev_pair);
    (void)hipStreamDestroy(h->bwd_owned);
    (void)hipStreamDestroy(h->wgrad_owned);
  }
  delete h;
  return DS_OK;
}

extern "C" int ds_stage_overlap_supported(const ds_stage* h) { return h && h->overlap_safe() ? 1 : 0; }

// Orders everything queued on the backward stream before whatever is queued next on the stage's stream.
static int stage_join(ds_stage* h) {
  if (h->bwd_stream && h->pair_valid) {  // what a paired pass queued on the stage's stream precedes what follows on the backward stream
    DS_CHECK_HIP(hipStreamWaitEvent(h->bwd_stream, h->ev_pair, 0));
    h->pair_valid = false;
  }
  DS_PROPAGATE(h->flush_deferred(true));
  if (h->bwd_stream && h->bwd_pending) {
    DS_CHECK_HIP(hipEventRecord(h->ev_join, h->bwd_stream));
    DS_CHECK_HIP(hipStreamWaitEvent(h->stream, h->ev_join, 0));
    h->bwd_pending = false;
  }
  return DS_OK;
}

extern "C" int ds_stage_enable_overlap(ds_stage* h, int on) {
  DS_CHECK_ARG(h != nullptr, "ds_stage_enable_overlap: null handle");
  if (on && !h->overlap_safe()) {
    ds_set_error("ds_stage_enable_overlap: this stage's forward and backward passes share workspace");
    return DS_EINVAL;
  }
  for (char f : h->slot_forwarded)
    if (f) { ds_set_error("ds_stage_enable_overlap: micro-batches in flight"); return DS_ESTATE; }
  DS_PROPAGATE(stage_join(h));
  if (!on) {
    h->bwd_stream = nullptr;
    h->wgrad_stream = nullptr;
    return DS_OK;
  }
  if (!h->bwd_owned) {
    DS_CHECK_HIP(hipStreamCreateWithFlags(&h->bwd_owned, hipStreamNonBlocking));
    DS_CHECK_HIP(hipStreamCreateWithFlags(&h->wgrad_owned, hipStreamNonBlocking));
    const int K = h->cfg.stash_slots;
    h->ev_forwarded.resize(K);
    h->ev_released.resize(K);
    for (int i = 0; i < K; ++i) {
      DS_CHECK_HIP(hipEventCreateWithFlags(&h->ev_forwarded[i], hipEventDisableTiming));
      DS_CHECK_HIP(hipEventCreateWithFlags(&h->ev_released[i], hipEventDisableTiming));
    }
    DS_CHECK_HIP(hipEventCreateWithFlags(&h->ev_join, hipEventDisableTiming));
    DS_CHECK_HIP(hipEventCreateWithFlags(&h->ev_dout, hipEventDisableTiming));
  }
  h->released_valid.assign(h->cfg.stash_slots, 0);  // everything queued so far is ordered on h->stream
  h->bwd_stream = h->bwd_owned;
  h->wgrad_stream = h->wgrad_owned;
  return DS_OK;
}

extern "C" int ds_stage_join(ds_stage* h) {
  DS_CHECK_ARG(h != nullptr, "ds_stage_join: null handle");
  return stage_join(h);
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
  DS_PROPAGATE(stage_join(h));  // a backward pass still queued reads the compute copies
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
  DS_PROPAGATE(ds_stage_acquire_slot(h, slot));
  const int rc = h->forward(slot, in, key_mask, out);
  if (rc == DS_OK) h->slot_forwarded[slot] = 1;
  if (rc == DS_OK && h->bwd_stream) DS_CHECK_HIP(hipEventRecord(h->ev_forwarded[slot], h->stream));
  return rc;
}

// F(fslot) and B(bslot) of different micro-batches in one call.  Stages that pair passes walk both chains together on
// the stage's stream (one grouped launch per level); the others get the two calls one after the other.
extern "C" int ds_stage_forward_backward(ds_stage* h, int fslot, const void* in, const float* key_mask, void* out, int bslot,
                                         const void* d_out, void* d_in) {
  DS_CHECK_ARG(h != nullptr && in != nullptr && out != nullptr && d_out != nullptr, "ds_stage_forward_backward: null argument");
  if (!h->pairs_passes()) {
    DS_PROPAGATE(ds_stage_forward(h, fslot, in, key_mask, out));
    return ds_stage_backward(h, bslot, d_out, d_in);
  }
  const int K = h->cfg.stash_slots;
  DS_CHECK_ARG(fslot >= 0 && fslot < K && bslot >= 0 && bslot < K && fslot != bslot,
               "ds_stage_forward_backward: slots %d and %d must be two different slots in [0,%d)", fslot, bslot, K);
  if (!h->bound) { ds_set_error("ds_stage_forward_backward: weights not bound"); return DS_ESTATE; }
  if (h->slot_forwarded[fslot]) {
    ds_set_error("ds_stage_forward_backward: slot %d still holds a micro-batch whose backward has not run", fslot);
    return DS_ESTATE;
  }
  if (!h->slot_forwarded[bslot]) {
    ds_set_error("ds_stage_forward_backward: slot %d holds no forwarded micro-batch", bslot);
    return DS_ESTATE;
  }
  DS_CHECK_ARG(ds_aligned16(in) && ds_aligned16(out) && ds_aligned16(d_out) && ds_aligned16(d_in),
               "ds_stage_forward_backward: in/out/d_out/d_in must be 16-byte aligned");
  if (h->bwd_stream && h->bwd_pending) {
    // the backward half shares its workspace with earlier backward passes: everything on the backward stream first
    DS_CHECK_HIP(hipEventRecord(h->ev_join, h->bwd_stream));
    DS_CHECK_HIP(hipStreamWaitEvent(h->stream, h->ev_join, 0));
  }
  DS_PROPAGATE(ds_stage_acquire_slot(h, fslot));
  const int rc = h->forward_backward(fslot, in, key_mask, out, bslot, d_out, d_in);
  if (rc != DS_OK) return rc;
  h->slot_forwarded[fslot] = 1;
  h->slot_forwarded[bslot] = 0;
  if (h->bwd_stream) {
    DS_CHECK_HIP(hipEventRecord(h->ev_forwarded[fslot], h->stream));
    DS_CHECK_HIP(hipEventRecord(h->ev_released[bslot], h->stream));
    h->released_valid[bslot] = 1;
    h->bwd_pending = true;  // ds_stage_join orders the weight-gradient stream behind the backward stream, and that before the caller
    // a backward pass issued on its own after this call runs on the backward stream and reuses this pass's workspace
    if (!h->ev_pair) DS_CHECK_HIP(hipEventCreateWithFlags(&h->ev_pair, hipEventDisableTiming));
    DS_CHECK_HIP(hipEventRecord(h->ev_pair, h->stream));
    h->pair_valid = true;
  }
  return DS_OK;
}

// after: 0 = the producer of d_out is whatever has been queued on the stage's stream so far; 1 = `ready` (an event, or
// NULL for "already complete / ordered before F(slot)") says when d_out may be read
static int stage_backward(ds_stage* h, int slot, const void* d_out, void* d_in, int after, hipEvent_t ready) {
  DS_CHECK_ARG(h != nullptr && d_out != nullptr, "ds_stage_backward: null argument");
  DS_CHECK_ARG(slot >= 0 && slot < h->cfg.stash_slots, "ds_stage_backward: slot %d out of range [0,%d)", slot, h->cfg.stash_slots);
  if (!h->slot_forwarded[slot]) {
    ds_set_error("ds_stage_backward: slot %d holds no forwarded micro-batch", slot);
    return DS_ESTATE;
  }
  DS_CHECK_ARG(ds_aligned16(d_out) && ds_aligned16(d_in), "ds_stage_backward: d_out/d_in must be 16-byte aligned");
  int rc;
  if (h->bwd_stream) {
    DS_CHECK_HIP(hipStreamWaitEvent(h->bwd_stream, h->ev_forwarded[slot], 0));
    if (h->pair_valid) {
      DS_CHECK_HIP(hipStreamWaitEvent(h->bwd_stream, h->ev_pair, 0));
      h->pair_valid = false;  // the backward stream is behind it from here on
    }
    if (!after) {
      DS_CHECK_HIP(hipEventRecord(h->ev_dout, h->stream));
      DS_CHECK_HIP(hipStreamWaitEvent(h->bwd_stream, h->ev_dout, 0));
    } else if (ready) {
      DS_CHECK_HIP(hipStreamWaitEvent(h->bwd_stream, ready, 0));
    }
    hipStream_t fwd = h->stream;
    h->stream = h->bwd_stream;
    rc = h->backward(slot, d_out, d_in);
    h->stream = fwd;
    (void)hipEventRecord(h->ev_released[slot], h->bwd_stream);
    h->released_valid[slot] = 1;
    h->bwd_pending = true;
  } else {
    if (after && ready) DS_CHECK_HIP(hipStreamWaitEvent(h->stream, ready, 0));
    rc = h->backward(slot, d_out, d_in);
  }
  h->slot_forwarded[slot] = 0;
  return rc;
}

extern "C" int ds_stage_backward(ds_stage* h, int slot, const void* d_out, void* d_in) {
  return stage_backward(h, slot, d_out, d_in, 0, nullptr);
}

extern "C" int ds_stage_backward_after(ds_stage* h, int slot, const void* d_out, void* d_in, void* ready_event) {
  return stage_backward(h, slot, d_out, d_in, 1, (hipEvent_t)ready_event);
}

extern "C" void* ds_stage_backward_event(ds_stage* h, int slot) {
  if (!h || slot < 0 || slot >= h->cfg.stash_slots || !h->bwd_stream || !h->released_valid[slot]) return nullptr;
  return (void*)h->ev_released[slot];
}

extern "C" int ds_stage_wait_backward(ds_stage* h, int slot, void* stream) {
  DS_CHECK_ARG(h != nullptr, "ds_stage_wait_backward: null handle");
  DS_CHECK_ARG(slot >= 0 && slot < h->cfg.stash_slots, "ds_stage_wait_backward: slot %d out of range [0,%d)", slot, h->cfg.stash_slots);
  if (h->bwd_stream && h->released_valid[slot]) DS_CHECK_HIP(hipStreamWaitEvent((hipStream_t)stream, h->ev_released[slot], 0));
  else if ((hipStream_t)stream != h->stream) {
    // one stream: the pass is ordered on the stage's stream; another stream waits for what is queued there
    hipEvent_t e = nullptr;
    DS_CHECK_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    DS_CHECK_HIP(hipEventRecord(e, h->stream));
    DS_CHECK_HIP(hipStreamWaitEvent((hipStream_t)stream, e, 0));
    DS_CHECK_HIP(hipEventDestroy(e));
  }
  return DS_OK;
}

extern "C" int ds_stage_release_slot(ds_stage* h, int slot) {
  DS_CHECK_ARG(h != nullptr, "ds_stage_release_slot: null handle");
  DS_CHECK_ARG(slot >= 0 && slot < h->cfg.stash_slots, "ds_stage_release_slot: slot %d out of range [0,%d)", slot, h->cfg.stash_slots);
  if (!h->slot_forwarded[slot]) {
    ds_set_error("ds_stage_release_slot: slot %d holds no forwarded micro-batch", slot);
    return DS_ESTATE;
  }
  DS_PROPAGATE(h->release(slot));
  h->slot_forwarded[slot] = 0;
  return DS_OK;
}

extern "C" size_t ds_stage_workspace_bytes(const ds_stage* h) { return h ? h->workspace_bytes() : 0; }
extern "C" size_t ds_stage_stash_bytes(const ds_stage* h, int slots) { return h ? h->stash_bytes(slots) : 0; }

extern "C" int ds_stage_sync(ds_stage* h) {
  DS_CHECK_ARG(h != nullptr, "ds_stage_sync: null handle");
  DS_PROPAGATE(stage_join(h));
  DS_CHECK_HIP(hipStreamSynchronize(h->stream));
  return DS_OK;
}
