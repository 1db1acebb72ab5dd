// Library-wide pieces of the artk C-ABI: error string and version.
#include "common.hpp"

#include <mutex>
#include <vector>

namespace artk {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// ---- profiling -------------------------------------------------------------
struct ProfRec {
  hipEvent_t a, b;
  int kind;
};
static std::vector<ProfRec> g_recs;
static std::mutex g_prof_mu;
static bool g_prof_on = false;
static hipEvent_t g_open[PROF_KINDS];

void prof_begin(int kind, hipStream_t st) {
  if (!g_prof_on) return;
  std::lock_guard<std::mutex> lk(g_prof_mu);
  hipEvent_t e;
  if (hipEventCreate(&e) != hipSuccess) return;
  (void)hipEventRecord(e, st);
  g_open[kind] = e;
}

void prof_end(int kind, hipStream_t st) {
  if (!g_prof_on) return;
  std::lock_guard<std::mutex> lk(g_prof_mu);
  if (g_open[kind] == nullptr) return;
  hipEvent_t e;
  if (hipEventCreate(&e) != hipSuccess) return;
  (void)hipEventRecord(e, st);
  g_recs.push_back({g_open[kind], e, kind});
  g_open[kind] = nullptr;
}
}  // namespace artk

extern "C" {
int32_t artk_profile_enable(int32_t on) {
  std::lock_guard<std::mutex> lk(artk::g_prof_mu);
  for (auto& r : artk::g_recs) {
    (void)hipEventDestroy(r.a);
    (void)hipEventDestroy(r.b);
  }
  artk::g_recs.clear();
  for (auto& e : artk::g_open) e = nullptr;
  artk::g_prof_on = on != 0;
  return ARTK_OK;
}

int32_t artk_profile_collect(int32_t kind, double* total_ms, int64_t* launches) {
  std::lock_guard<std::mutex> lk(artk::g_prof_mu);
  double t = 0.0;
  int64_t n = 0;
  for (auto& r : artk::g_recs) {
    if (r.kind != kind) continue;
    float ms = 0.f;
    hipError_t e = hipEventElapsedTime(&ms, r.a, r.b);
    if (e != hipSuccess) {
      artk::set_error("hipEventElapsedTime failed: %s (synchronise before collecting)",
                      hipGetErrorString(e));
      return (int32_t)e;
    }
    t += ms;
    ++n;
  }
  if (total_ms) *total_ms = t;
  if (launches) *launches = n;
  return ARTK_OK;
}

int32_t artk_abi_version(void) { return 4; }
const char* artk_last_error(void) { return artk::g_err; }
}
