// Error channel and the optional per-kernel timer of the library.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>
#include "ody_common.h"

namespace {
thread_local char g_err[512] = "";

struct Span { const char* name; hipEvent_t start, stop; };
std::mutex g_mu;
bool g_profile = false;
std::vector<Span> g_spans;
constexpr size_t kMaxSpans = 1u << 18;   // launches kept between two ody_profile_collect calls
}  // namespace

void ody_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int ody_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    ody_set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return ODY_ERR_LAUNCH;
  }
  return ODY_OK;
}

int ody_allow_dynamic_lds(const void* kernel, size_t bytes, const char* who) {
  static std::mutex mu;
  static std::vector<std::pair<const void*, int>> done;   // (kernel, device) pairs already raised
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    ody_set_error("%s: no current HIP device", who);
    return ODY_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> lk(mu);
  for (const auto& kd : done)
    if (kd.first == kernel && kd.second == dev) return ODY_OK;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) {
    ody_set_error("%s: hipFuncSetAttribute(%zu bytes of dynamic LDS) failed: %s", who, bytes, hipGetErrorString(e));
    return ODY_ERR_LAUNCH;
  }
  done.emplace_back(kernel, dev);
  return ODY_OK;
}

OdyKernelScope::OdyKernelScope(const char* name, hipStream_t st) : name_(name), st_(st), start_(nullptr) {
  if (!g_profile) return;
  if (hipEventCreate(&start_) != hipSuccess) { start_ = nullptr; return; }
  (void)hipEventRecord(start_, st_);
}

OdyKernelScope::~OdyKernelScope() {
  if (!start_) return;
  hipEvent_t stop;
  if (hipEventCreate(&stop) != hipSuccess) { (void)hipEventDestroy(start_); return; }
  (void)hipEventRecord(stop, st_);
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_spans.size() >= kMaxSpans) {   // nobody collects: drop the span instead of growing without bound
    (void)hipEventDestroy(start_);
    (void)hipEventDestroy(stop);
    return;
  }
  g_spans.push_back({name_, start_, stop});
}

extern "C" const char* ody_last_error(void) { return g_err; }
extern "C" int ody_version(void) { return 1; }

extern "C" int ody_device_info(int* compute_units, int* clock_khz, int* lds_bytes_per_cu) {
  int dev = 0, v = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    ody_set_error("ody_device_info: no current HIP device");
    return ODY_ERR_LAUNCH;
  }
  const hipDeviceAttribute_t what[3] = {hipDeviceAttributeMultiprocessorCount, hipDeviceAttributeClockRate,
                                        hipDeviceAttributeMaxSharedMemoryPerMultiprocessor};
  int* const where[3] = {compute_units, clock_khz, lds_bytes_per_cu};
  for (int k = 0; k < 3; k++) {
    if (!where[k]) continue;
    if (hipDeviceGetAttribute(&v, what[k], dev) != hipSuccess) {
      ody_set_error("ody_device_info: hipDeviceGetAttribute failed");
      return ODY_ERR_LAUNCH;
    }
    *where[k] = v;
  }
  return ODY_OK;
}

extern "C" int ody_profile_enable(int on) {
  std::lock_guard<std::mutex> lk(g_mu);
  g_profile = on != 0;
  return ODY_OK;
}

extern "C" int ody_profile_collect(char* out, size_t cap) {
  std::vector<Span> spans;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    spans.swap(g_spans);
  }
  struct Agg { int n = 0; double total = 0, mn = 1e30; };
  std::map<std::string, Agg> agg;
  for (auto& s : spans) {
    float ms = 0.f;
    if (hipEventSynchronize(s.stop) == hipSuccess && hipEventElapsedTime(&ms, s.start, s.stop) == hipSuccess) {
      Agg& a = agg[s.name];
      a.n++;
      a.total += ms;
      if (ms < a.mn) a.mn = ms;
    }
    (void)hipEventDestroy(s.start);
    (void)hipEventDestroy(s.stop);
  }
  std::string txt;
  char line[256];
  for (auto& kv : agg) {
    snprintf(line, sizeof(line), "%s %d %.6f %.6f\n", kv.first.c_str(), kv.second.n, kv.second.total, kv.second.mn);
    txt += line;
  }
  if (!out || cap == 0) return ODY_ERR_NULL;
  if (txt.size() + 1 > cap) {
    ody_set_error("ody_profile_collect: buffer of %zu bytes, %zu needed", cap, txt.size() + 1);
    return ODY_ERR_WORKSPACE;
  }
  memcpy(out, txt.c_str(), txt.size() + 1);
  return ODY_OK;
}
