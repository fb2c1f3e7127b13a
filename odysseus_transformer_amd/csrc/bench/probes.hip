// Measurement aids of bench.py, built into their own library (lib/libodysseus_bench.so): synthetic kernels that
// say what the matrix pipe sustains and what the ingredients of an attention tile cost.  Nothing on the hot path
// uses them and the product library does not contain them.
#include <hip/hip_runtime.h>
#include <mutex>
#include <stdint.h>
#include <stdio.h>

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

enum { PROBE_OK = 0, PROBE_ERR_ARG = -1, PROBE_ERR_LAUNCH = -6 };
enum ody_probe_parts { ODY_PROBE_VECTOR = 1, ODY_PROBE_LDS_READS = 2, ODY_PROBE_DIRECT_LOADS = 4 };

#define PROBE_REQUIRE(cond, ...)                 \
  do {                                           \
    if (!(cond)) {                               \
      fprintf(stderr, __VA_ARGS__);              \
      fputc('\n', stderr);                       \
      return PROBE_ERR_ARG;                      \
    }                                            \
  } while (0)

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return PROBE_OK;
  fprintf(stderr, "%s: launch failed: %s\n", what, hipGetErrorString(e));
  return PROBE_ERR_LAUNCH;
}
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float ody_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---------------------------------------------------------------------------
// MFMA-only loops on register operands: the sustained rate of the matrix pipe for given operand data, with
// either bf16 instruction shape.  shape 0: v_mfma_f32_32x32x16_bf16, 16 accumulator tiles (a 128 x 128 wavefront
// tile, k = 16 per iteration); shape 1: v_mfma_f32_16x16x32_bf16, 64 accumulator tiles (the same tile, k = 32 per
// iteration).  4 wavefronts per block; FLOP = blocks * 4 * iters * 16 * 32768 for shape 0, twice that for shape 1.
// ---------------------------------------------------------------------------
namespace {
template <int SHAPE>
__global__ __launch_bounds__(256) void mfma_probe_kernel(const bf16x8* __restrict__ in, float* __restrict__ sink,
                                                         int iters) {
  const int tid = blockIdx.x * 256 + threadIdx.x;
  float s = 0.f;
  if (SHAPE == 0) {
    bf16x8 a[4], b[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      a[j] = in[(tid * 16 + j) & 0xffff];
      b[j] = in[(tid * 16 + 8 + j) & 0xffff];
    }
    f32x16 c[4][4] = {};
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int x = 0; x < 4; x++)
#pragma unroll
        for (int y = 0; y < 4; y++) c[x][y] = mfma32(a[x], b[y], c[x][y]);
    }
#pragma unroll
    for (int x = 0; x < 4; x++)
#pragma unroll
      for (int y = 0; y < 4; y++)
#pragma unroll
        for (int r = 0; r < 16; r++) s += c[x][y][r];
  } else {
    bf16x8 a[8], b[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      a[j] = in[(tid * 16 + j) & 0xffff];
      b[j] = in[(tid * 16 + 8 + j) & 0xffff];
    }
    f32x4 c[8][8] = {};
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int x = 0; x < 8; x++)
#pragma unroll
        for (int y = 0; y < 8; y++) c[x][y] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[x], b[y], c[x][y], 0, 0, 0);
    }
#pragma unroll
    for (int x = 0; x < 8; x++)
#pragma unroll
      for (int y = 0; y < 8; y++)
#pragma unroll
        for (int r = 0; r < 4; r++) s += c[x][y][r];
  }
  sink[tid] = s;
}
}  // namespace

// operands: at least 1 MiB of bf16 on the device; sink: blocks * 256 floats
extern "C" int ody_bench_mfma_probe(const void* operands, float* sink, int blocks, int iters, int shape, void* stream) {
  PROBE_REQUIRE(operands && sink, "ody_bench_mfma_probe: NULL pointer");
  PROBE_REQUIRE(blocks > 0 && iters > 0 && (shape == 0 || shape == 1), "ody_bench_mfma_probe: blocks=%d iters=%d shape=%d",
                blocks, iters, shape);
  PROBE_REQUIRE(aligned16(operands), "ody_bench_mfma_probe: operands must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (shape == 0)
    hipLaunchKernelGGL(mfma_probe_kernel<0>, dim3(blocks), dim3(256), 0, st, static_cast<const bf16x8*>(operands), sink, iters);
  else
    hipLaunchKernelGGL(mfma_probe_kernel<1>, dim3(blocks), dim3(256), 0, st, static_cast<const bf16x8*>(operands), sink, iters);
  return check_launch("mfma_probe");
}

// ---------------------------------------------------------------------------
// What each ingredient of an attention tile costs on top of the bare MFMAs: 8 wavefronts (two per SIMD),
// one workgroup per CU, a workgroup barrier per turn; per turn and wavefront 32 MFMAs, then -- as asked --
// the vector work of a 32 x 64 score tile (exp2, row sum, bf16 packing), the MFMA A operands read from LDS
// (one 16-byte read per lane and MFMA), and this wavefront's share (4 of 32) of the 16-byte direct loads that
// bring the next 32 KB into a three-stage LDS ring (from the 64 MiB at stream_src).  Built combinations of
// ody_probe_parts: 0, 1, 3, 5, 7.  operands: at least 1 MiB of bf16; sink: blocks * 512 floats.
// FLOP: blocks * 8 * turns * 32 * 32768.
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
  static std::mutex mu;
  {
    std::lock_guard<std::mutex> lk(mu);   // the LDS opt-in is per device; asking again is harmless
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&pipeline_probe_kernel<WHAT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      fprintf(stderr, "pipeline_probe: cannot opt in to %zu bytes of LDS: %s\n", smem, hipGetErrorString(e));
      return PROBE_ERR_LAUNCH;
    }
  }
  hipLaunchKernelGGL(pipeline_probe_kernel<WHAT>, dim3(blocks), dim3(512), smem, st, static_cast<const bf16x8*>(operands),
                     static_cast<const char*>(src), sink, turns);
  return check_launch("pipeline_probe");
}
}  // namespace

extern "C" int ody_bench_pipeline_probe(const void* operands, const void* stream_src, float* sink, int blocks, int turns,
                                  int what, void* stream) {
  PROBE_REQUIRE(operands && sink, "ody_bench_pipeline_probe: NULL pointer");
  PROBE_REQUIRE(blocks > 0 && turns > 0, "ody_bench_pipeline_probe: blocks=%d turns=%d", blocks, turns);
  PROBE_REQUIRE(aligned16(operands), "ody_bench_pipeline_probe: operands must be 16-byte aligned");
  PROBE_REQUIRE(!(what & ODY_PROBE_DIRECT_LOADS) || (stream_src && aligned16(stream_src)),
                "ody_bench_pipeline_probe: direct loads need a 16-byte aligned stream_src of 64 MiB");
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
      fprintf(stderr, "ody_bench_pipeline_probe: combination %d is not built (0, 1, 3, 5, 7 are)\n", what);
      return PROBE_ERR_ARG;
  }
}
