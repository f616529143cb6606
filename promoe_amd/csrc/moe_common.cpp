#include "moe_common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_err[512] = "";

void moe_set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
}

extern "C" const char *moe_last_error(void) { return g_err; }

int moe_check_hip(hipError_t e, const char *what) {
  if (e == hipSuccess) return MOE_OK;
  moe_set_error("%s: %s", what, hipGetErrorString(e));
  return MOE_EHIP;
}

int moe_check_launch(const char *what) { return moe_check_hip(hipGetLastError(), what); }

// ---- per-kernel timing -----------------------------------------------------
#include <mutex>
#include <vector>
namespace {
struct KRec { int kid; hipEvent_t a, b; };
std::mutex g_kt_mu;
bool g_kt_on = false;
std::vector<KRec> g_kt_recs;
std::vector<hipEvent_t> g_kt_free;
hipEvent_t g_kt_open[MOE_K_COUNT];
const size_t kMaxRecs = 1 << 15;
hipEvent_t kt_event() {
  if (!g_kt_free.empty()) { hipEvent_t e = g_kt_free.back(); g_kt_free.pop_back(); return e; }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}
}  // namespace

void moe_ktimer_begin(int kid, hipStream_t s) {
  if (!g_kt_on) return;
  std::lock_guard<std::mutex> lk(g_kt_mu);
  if (g_kt_recs.size() >= kMaxRecs) return;
  hipEvent_t e = kt_event();
  if (!e) return;
  (void)hipEventRecord(e, s);
  g_kt_open[kid] = e;
}
void moe_ktimer_end(int kid, hipStream_t s) {
  if (!g_kt_on) return;
  std::lock_guard<std::mutex> lk(g_kt_mu);
  if (!g_kt_open[kid]) return;
  hipEvent_t e = kt_event();
  if (!e) return;
  (void)hipEventRecord(e, s);
  g_kt_recs.push_back(KRec{kid, g_kt_open[kid], e});
  g_kt_open[kid] = nullptr;
}

extern "C" int moe_kernel_timing(int enable) {
  std::lock_guard<std::mutex> lk(g_kt_mu);
  g_kt_on = enable != 0;
  for (auto &r : g_kt_recs) { g_kt_free.push_back(r.a); g_kt_free.push_back(r.b); }
  g_kt_recs.clear();
  for (auto &e : g_kt_open) e = nullptr;
  return MOE_OK;
}

extern "C" int moe_kernel_timing_read(int kernel_id, double *total_ms, int *calls) {
  if (kernel_id < 0 || kernel_id >= MOE_K_COUNT || !total_ms || !calls) { moe_set_error("moe_kernel_timing_read: bad argument"); return MOE_EINVAL; }
  std::lock_guard<std::mutex> lk(g_kt_mu);
  double tot = 0;
  int n = 0;
  for (auto &r : g_kt_recs) {
    if (r.kid != kernel_id) continue;
    if (hipEventSynchronize(r.b) != hipSuccess) continue;
    float ms = 0;
    if (hipEventElapsedTime(&ms, r.a, r.b) == hipSuccess) { tot += ms; ++n; }
  }
  *total_ms = tot;
  *calls = n;
  return MOE_OK;
}
