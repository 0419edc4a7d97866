// Version and error reporting for the C ABI.
#include "fsa_common.h"

#include <mutex>
#include <vector>

namespace fsa {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

struct ProfRec {
  const char* name;
  hipEvent_t start, stop;
};
static std::mutex g_prof_mu;
static bool g_prof_on = false;
static std::vector<ProfRec> g_prof;

ProfScope::ProfScope(const char* name, hipStream_t stream) : idx_(-1), stream_(stream) {
  if (!g_prof_on) return;
  std::lock_guard<std::mutex> lk(g_prof_mu);
  ProfRec r;
  r.name = name;
  if (hipEventCreate(&r.start) != hipSuccess || hipEventCreate(&r.stop) != hipSuccess) return;
  (void)hipEventRecord(r.start, stream);
  g_prof.push_back(r);
  idx_ = (int)g_prof.size() - 1;
}

ProfScope::~ProfScope() {
  if (idx_ < 0) return;
  std::lock_guard<std::mutex> lk(g_prof_mu);
  (void)hipEventRecord(g_prof[idx_].stop, stream_);
}
}  // namespace fsa

extern "C" int fsa_version(void) { return 100; }
extern "C" const char* fsa_last_error(void) { return fsa::g_err; }

extern "C" int fsa_profile_enable(int on) {
  std::lock_guard<std::mutex> lk(fsa::g_prof_mu);
  for (auto& r : fsa::g_prof) {
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  fsa::g_prof.clear();
  fsa::g_prof_on = on != 0;
  return 0;
}

extern "C" int fsa_profile_count(void) {
  std::lock_guard<std::mutex> lk(fsa::g_prof_mu);
  return (int)fsa::g_prof.size();
}

extern "C" int fsa_profile_get(int i, char* name, int name_cap, float* ms) {
  std::lock_guard<std::mutex> lk(fsa::g_prof_mu);
  if (i < 0 || i >= (int)fsa::g_prof.size() || !name || name_cap <= 0 || !ms) {
    fsa::set_error("fsa_profile_get: bad index or buffer");
    return FSA_ERR_INVALID;
  }
  fsa::ProfRec& r = fsa::g_prof[i];
  hipError_t e = hipEventSynchronize(r.stop);
  if (e == hipSuccess) e = hipEventElapsedTime(ms, r.start, r.stop);
  if (e != hipSuccess) {
    fsa::set_error("fsa_profile_get: %s", hipGetErrorString(e));
    return (int)e;
  }
  snprintf(name, name_cap, "%s", r.name);
  return 0;
}
