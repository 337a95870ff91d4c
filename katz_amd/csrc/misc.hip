// ABI version and error strings of the katz_hip C ABI.
#include "kh_common.h"

#include <mutex>
#include <vector>

namespace {
struct ProfEntry { int tag; hipEvent_t start, stop; };
std::mutex g_prof_mu;
std::vector<ProfEntry> g_prof;
bool g_prof_on = false;
}  // namespace

bool kh_prof_enabled() { return g_prof_on; }

void kh_prof_events(int tag, hipEvent_t* start, hipEvent_t* stop) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  ProfEntry e;
  e.tag = tag;
  (void)hipEventCreate(&e.start);
  (void)hipEventCreate(&e.stop);
  g_prof.push_back(e);
  *start = e.start;
  *stop = e.stop;
}

KH_EXPORT int kh_profile_begin(void) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  for (auto& e : g_prof) { (void)hipEventDestroy(e.start); (void)hipEventDestroy(e.stop); }
  g_prof.clear();
  g_prof_on = true;
  return KH_OK;
}

// Stops profiling, waits for the recorded launches, writes (tag, milliseconds) per launch in launch
// order.  Returns the number of launches recorded (may exceed capacity; only capacity are written),
// or a negative hipError_t.
KH_EXPORT int kh_profile_end(int32_t* tags, float* ms, int capacity) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  g_prof_on = false;
  int n = 0;
  int rc = 0;
  for (auto& e : g_prof) {
    if (rc == 0) {
      hipError_t err = hipEventSynchronize(e.stop);
      float t = 0.f;
      if (err == hipSuccess) err = hipEventElapsedTime(&t, e.start, e.stop);
      if (err != hipSuccess) rc = -(int)err;
      if (n < capacity && tags && ms) { tags[n] = e.tag; ms[n] = t; }
    }
    ++n;
    (void)hipEventDestroy(e.start);
    (void)hipEventDestroy(e.stop);
  }
  g_prof.clear();
  return rc != 0 ? rc : n;
}

KH_EXPORT int kh_version(void) { return 2; }

KH_EXPORT const char* kh_error_string(int code) {
  switch (code) {
    case KH_OK: return "ok";
    case KH_ERR_INVALID_ARG: return "katz_hip: invalid argument (null pointer, non-positive size or inconsistent shape)";
    case KH_ERR_UNSUPPORTED: return "katz_hip: shape not supported by the kernels";
    case KH_ERR_ALIGNMENT: return "katz_hip: pointer or stride not 16-byte aligned";
    case KH_ERR_TOO_LARGE: return "katz_hip: size beyond the documented maximum";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "katz_hip: unknown error code";
}
