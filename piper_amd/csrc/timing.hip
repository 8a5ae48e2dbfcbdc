// Optional per-kernel timing with HIP events on the launch stream.  Off by default; when on,
// every kernel launch of the library is bracketed by two event records (a few microseconds of
// host time each, nothing on the device besides the timestamps).
#include "pk_common.h"
#include <mutex>
#include <vector>

namespace pk_timing {

namespace {
struct Rec { int id; hipEvent_t start, stop; };
std::mutex g_mu;
bool g_on = false;
int g_only = -1;   // >= 0: only launches of this kernel id are bracketed
std::vector<Rec> g_recs;
std::vector<hipEvent_t> g_pool;

hipEvent_t get_event() {
  if (!g_pool.empty()) { hipEvent_t e = g_pool.back(); g_pool.pop_back(); return e; }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}
}  // namespace

const char* const kNames[K_COUNT] = {
    "gate_logits", "route_topk", "route_topk_bwd", "gate_logits_bwd", "sort_hist", "sort_scan",
    "sort_scatter", "counts_to_starts", "permute_fwd", "gather_reduce", "combine_bwd",
    "swiglu_gate_up", "swiglu_down", "swiglu_dgrad_dh", "swiglu_dgrad_dx", "swiglu_wgrad",
    "simt_gemm", "swiglu_elementwise", "bucket_pack", "bucket_unpack", "bucket_zero", "adamw",
    "rmsnorm_fwd", "rmsnorm_bwd", "misc", "swiglu_wgrad_w2", "swiglu_wgrad_w13"};

Scope::Scope(int id, hipStream_t s) : stream_(s), slot_(-1) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (!g_on || (g_only >= 0 && id != g_only)) return;
  Rec r{id, get_event(), get_event()};
  if (!r.start || !r.stop) return;
  if (hipEventRecord(r.start, s) != hipSuccess) return;
  g_recs.push_back(r);
  slot_ = (int)g_recs.size() - 1;
}
Scope::~Scope() {
  if (slot_ < 0) return;
  std::lock_guard<std::mutex> lk(g_mu);
  if (slot_ < (int)g_recs.size()) (void)hipEventRecord(g_recs[slot_].stop, stream_);
}

}  // namespace pk_timing

extern "C" {

int pk_timing_enable(int on) {
  std::lock_guard<std::mutex> lk(pk_timing::g_mu);
  pk_timing::g_on = on != 0;
  return PK_OK;
}

int64_t pk_timing_collect(int32_t* ids, float* ms, int64_t max_records) {
  std::lock_guard<std::mutex> lk(pk_timing::g_mu);
  int64_t n = 0;
  for (auto& r : pk_timing::g_recs) {
    float t = 0.f;
    if (hipEventSynchronize(r.stop) == hipSuccess && hipEventElapsedTime(&t, r.start, r.stop) == hipSuccess) {
      if (n < max_records && ids && ms) { ids[n] = r.id; ms[n] = t; }
      ++n;
    }
    pk_timing::g_pool.push_back(r.start);
    pk_timing::g_pool.push_back(r.stop);
  }
  pk_timing::g_recs.clear();
  return n;
}

int pk_timing_select(int kernel_id) {
  std::lock_guard<std::mutex> lk(pk_timing::g_mu);
  pk_timing::g_only = (kernel_id >= 0 && kernel_id < pk_timing::K_COUNT) ? kernel_id : -1;
  return PK_OK;
}

const char* pk_timing_kernel_name(int id) {
  return (id >= 0 && id < pk_timing::K_COUNT) ? pk_timing::kNames[id] : "unknown";
}

}  // extern "C"
