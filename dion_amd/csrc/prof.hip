#include "prof.h"
#include "../../include/dion_amd.h"
#include <vector>
#include <mutex>
#include <atomic>

namespace {
struct Rec { hipEvent_t a, b; int kind; double work; };
std::mutex g_mu;
std::atomic<bool> g_on{false};   // read by every launch, from any host thread
std::vector<Rec> g_recs;
}  // namespace

DaProfScope::DaProfScope(int kind, double work, hipStream_t stream) : slot(-1), s(stream) {
  if (!g_on.load(std::memory_order_relaxed)) return;
  std::lock_guard<std::mutex> lk(g_mu);
  Rec r{};
  r.kind = kind; r.work = work;
  if (hipEventCreate(&r.a) != hipSuccess || hipEventCreate(&r.b) != hipSuccess) return;
  (void)hipEventRecord(r.a, stream);
  slot = (int)g_recs.size();
  g_recs.push_back(r);
}

DaProfScope::~DaProfScope() {
  if (slot < 0) return;
  std::lock_guard<std::mutex> lk(g_mu);
  (void)hipEventRecord(g_recs[slot].b, s);
}

extern "C" {

int dion_amd_profile_enable(int on) {
  std::lock_guard<std::mutex> lk(g_mu);
  g_on.store(on != 0, std::memory_order_relaxed);
  return 0;
}

int dion_amd_profile_reset(void) {
  std::lock_guard<std::mutex> lk(g_mu);
  for (auto& r : g_recs) { (void)hipEventDestroy(r.a); (void)hipEventDestroy(r.b); }
  g_recs.clear();
  return 0;
}

int dion_amd_profile_read(int kind, long long* launches, double* total_ms, double* total_work) {
  if (kind < 0 || kind >= DA_PROF_KINDS || !launches || !total_ms || !total_work) return DION_AMD_ERR_ARG;
  std::lock_guard<std::mutex> lk(g_mu);
  long long n = 0;
  double ms = 0.0, work = 0.0;
  for (auto& r : g_recs) {
    if (r.kind != kind) continue;
    hipError_t e = hipEventSynchronize(r.b);
    if (e != hipSuccess) return (int)e;
    float t = 0.f;
    e = hipEventElapsedTime(&t, r.a, r.b);
    if (e != hipSuccess) return (int)e;
    ++n; ms += t; work += r.work;
  }
  *launches = n; *total_ms = ms; *total_work = work;
  return 0;
}

}  // extern "C"
