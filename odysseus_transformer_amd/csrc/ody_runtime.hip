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

// ---------------------------------------------------------------------------
// MFMA-only loop on register operands: the sustained rate of the matrix pipe for given operand data
// ---------------------------------------------------------------------------
namespace {
__global__ __launch_bounds__(256) void mfma_probe_kernel(const bf16x8* __restrict__ in, float* __restrict__ sink,
                                                         int iters) {
  const int tid = blockIdx.x * 256 + threadIdx.x;
  bf16x8 a[4], b[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    a[j] = in[(tid * 8 + j) & 0xffff];
    b[j] = in[(tid * 8 + 4 + j) & 0xffff];
  }
  f32x16 c[4];
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int r = 0; r < 16; r++) c[j][r] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 4; u++)
#pragma unroll
      for (int j = 0; j < 4; j++) c[j] = mfma32(a[(u + j) & 3], b[u], c[j]);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int r = 0; r < 16; r++) s += c[j][r];
  sink[tid] = s;
}
}  // namespace

extern "C" int ody_mfma_probe(const void* operands, float* sink, int blocks, int iters, void* stream) {
  ODY_REQUIRE(operands && sink, ODY_ERR_NULL, "ody_mfma_probe: NULL pointer");
  ODY_REQUIRE(blocks > 0 && iters > 0, ODY_ERR_BAD_SHAPE, "ody_mfma_probe: blocks=%d iters=%d", blocks, iters);
  ODY_REQUIRE(ody_aligned16(operands), ODY_ERR_MISALIGNED, "ody_mfma_probe: operands must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  ODY_LAUNCH("mfma_probe", st, mfma_probe_kernel, dim3(blocks), dim3(256), 0, static_cast<const bf16x8*>(operands), sink,
             iters);
  return ody_check_launch("mfma_probe");
}

// ---------------------------------------------------------------------------
// What each ingredient of an attention tile costs on top of the bare MFMAs: 8 wavefronts (two per SIMD),
// one workgroup per CU, a workgroup barrier per turn; per turn and wavefront 32 MFMAs, then -- as asked --
// the vector work of a 32 x 64 score tile (exp2, row sum, bf16 packing), the MFMA A operands read from LDS
// (one 16-byte read per lane and MFMA), and this wavefront's share (4 of 32) of the 16-byte direct loads that
// bring the next 32 KB into a three-stage LDS ring.
// ---------------------------------------------------------------------------
namespace {
typedef __attribute__((address_space(3))) void* probe_lds_ptr;
typedef __attribute__((address_space(1))) const void* probe_global_ptr;

template <int WHAT>
__global__ __launch_bounds__(512) void pipeline_probe_kernel(const bf16x8* __restrict__ in, const char* __restrict__ src,
                                                             float* __restrict__ sink, int turns) {
  constexpr bool VEC = WHAT & ODY_PROBE_VECTOR, LDSR = WHAT & ODY_PROBE_LDS_READS, LOADS = WHAT & ODY_PROBE_DIRECT_LOADS;
  extern __shared__ __attribute__((aligned(16))) unsigned char probe_smem[];   // 3 stages of 32 KB
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  bf16x8* lds = reinterpret_cast<bf16x8*>(probe_smem);
  for (int q = tid; q < 6144; q += 512) lds[q] = in[(q * 7 + blockIdx.x) & 0xffff];
  bf16x8 a[4], pb[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    a[j] = in[(tid * 8 + j) & 0xffff];
    pb[j] = in[(tid * 8 + 4 + j) & 0xffff];
  }
  f32x16 acc[4], s[2];
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[j][r] = 0.f;
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int r = 0; r < 16; r++) s[j][r] = (float)a[j][r & 7] * 0.01f * (r + 1);
  float l4[4] = {0.f, 0.f, 0.f, 0.f};
  __syncthreads();
  for (int t = 0; t < turns; t++) {
    if (LOADS) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");   // the loads of two turns ago have landed
    __syncthreads();
    if (LOADS) {
      // every workgroup reads the same 32 KB in the same turn, as the query blocks of a head do with a K / V tile
      const char* from = src + ((size_t)(t & 2047) << 15);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int grp = 8 * j + wave;
        __builtin_amdgcn_global_load_lds((probe_global_ptr)(from + grp * 1024 + lane * 16),
                                         (probe_lds_ptr)(probe_smem + ((t + 2) % 3) * 32768 + grp * 1024), 16, 0, 0);
      }
    }
    if (LDSR) {
      const bf16x8* st = lds + (t % 3) * 2048;
      bf16x8 fr[4];
#pragma unroll
      for (int q = 0; q < 4; q++) fr[q] = st[q * 64 + lane];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < 32; q++) {
        acc[q & 3] = mfma32(fr[q & 3], pb[(q >> 2) & 3], acc[q & 3]);
        if (q + 4 < 32) fr[q & 3] = st[(q + 4) * 64 + lane];
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int q = 0; q < 32; q++) acc[q & 3] = mfma32(a[q & 3], pb[(q >> 2) & 3], acc[q & 3]);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (VEC) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float x = ody_exp2(fmaf(s[kt][r], 0.1f, -0.5f));
          l4[r & 3] += x;
          pb[2 * kt + (r >> 3)][r & 7] = (bf16)x;
        }
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("" : "+v"(s[0]), "+v"(s[1]));   // the scores count as new every turn
    }
  }
  if (LOADS) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  float r = (l4[0] + l4[1]) + (l4[2] + l4[3]);
#pragma unroll
  for (int j = 0; j < 4; j++) {
    r += (float)pb[j][0];
#pragma unroll
    for (int e = 0; e < 16; e++) r += acc[j][e];
  }
  sink[blockIdx.x * 512 + tid] = r;
}

template <int WHAT>
int launch_pipeline_probe(const void* operands, const void* src, float* sink, int blocks, int turns, hipStream_t st) {
  constexpr size_t smem = 3 * 32768;
  int rc = ody_allow_dynamic_lds(reinterpret_cast<const void*>(&pipeline_probe_kernel<WHAT>), smem, "pipeline_probe");
  if (rc) return rc;
  ODY_LAUNCH("pipeline_probe", st, pipeline_probe_kernel<WHAT>, dim3(blocks), dim3(512), smem,
             static_cast<const bf16x8*>(operands), static_cast<const char*>(src), sink, turns);
  return ody_check_launch("pipeline_probe");
}
}  // namespace

extern "C" int ody_pipeline_probe(const void* operands, const void* stream_src, float* sink, int blocks, int turns,
                                  int what, void* stream) {
  ODY_REQUIRE(operands && sink, ODY_ERR_NULL, "ody_pipeline_probe: NULL pointer");
  ODY_REQUIRE(blocks > 0 && turns > 0, ODY_ERR_BAD_SHAPE, "ody_pipeline_probe: blocks=%d turns=%d", blocks, turns);
  ODY_REQUIRE(ody_aligned16(operands), ODY_ERR_MISALIGNED, "ody_pipeline_probe: operands must be 16-byte aligned");
  ODY_REQUIRE(!(what & ODY_PROBE_DIRECT_LOADS) || (stream_src && ody_aligned16(stream_src)), ODY_ERR_NULL,
              "ody_pipeline_probe: direct loads need a 16-byte aligned stream_src of 64 MiB");
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (what) {
    case 0: return launch_pipeline_probe<0>(operands, stream_src, sink, blocks, turns, st);
    case ODY_PROBE_VECTOR: return launch_pipeline_probe<ODY_PROBE_VECTOR>(operands, stream_src, sink, blocks, turns, st);
    case ODY_PROBE_VECTOR | ODY_PROBE_LDS_READS:
      return launch_pipeline_probe<ODY_PROBE_VECTOR | ODY_PROBE_LDS_READS>(operands, stream_src, sink, blocks, turns, st);
    case ODY_PROBE_VECTOR | ODY_PROBE_DIRECT_LOADS:
      return launch_pipeline_probe<ODY_PROBE_VECTOR | ODY_PROBE_DIRECT_LOADS>(operands, stream_src, sink, blocks, turns, st);
    case ODY_PROBE_VECTOR | ODY_PROBE_LDS_READS | ODY_PROBE_DIRECT_LOADS:
      return launch_pipeline_probe<ODY_PROBE_VECTOR | ODY_PROBE_LDS_READS | ODY_PROBE_DIRECT_LOADS>(operands, stream_src, sink,
                                                                                                   blocks, turns, st);
    default:
      ody_set_error("ody_pipeline_probe: combination %d is not built (0, 1, 3, 5, 7 are)", what);
      return ODY_ERR_UNSUPPORTED;
  }
}
