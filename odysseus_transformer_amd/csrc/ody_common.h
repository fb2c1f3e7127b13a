// Shared device/host helpers for the gfx950 kernels of libodysseus_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "../../include/odysseus_hip.h"

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(2))) int i32x2;

#define ODY_LOG2E 1.4426950408889634f
#define ODY_LN2 0.6931471805599453f

// Sets the thread-local error string returned by ody_last_error().
void ody_set_error(const char* fmt, ...);
// Returns ODY_OK or ODY_ERR_LAUNCH after a kernel launch (reads hipGetLastError).
int ody_check_launch(const char* what);

// Raises a kernel's dynamic-LDS limit to `bytes` on the current device.  Done once per (kernel, device)
// under a lock, so concurrent first calls from several host threads and several devices are safe.
int ody_allow_dynamic_lds(const void* kernel, size_t bytes, const char* who);
// In-place rotation (inverse != 0: by the negative angle) of the first n_rot heads of a bf16 (rows, heads, D) array with
// the cos / sin table of ody_rope_table; s_row, s_h in elements.
int ody_launch_rope_from_table(void* x, const void* table, int64_t rows, int n_rot, int D, int64_t s_row, int64_t s_h,
                               int inverse, hipStream_t st);

// Brackets one kernel launch with a pair of HIP events on the launch stream when the
// timer is enabled (ody_profile_enable); costs one branch otherwise.
struct OdyKernelScope {
  OdyKernelScope(const char* name, hipStream_t st);
  ~OdyKernelScope();
  const char* name_;
  hipStream_t st_;
  hipEvent_t start_;
};

#define ODY_LAUNCH(name, st, kernel, grid, block, smem, ...)                      \
  do {                                                                            \
    OdyKernelScope ody_scope_(name, st);                                          \
    hipLaunchKernelGGL(kernel, grid, block, smem, st, __VA_ARGS__);               \
  } while (0)

#define ODY_REQUIRE(cond, code, ...)        \
  do {                                      \
    if (!(cond)) {                          \
      ody_set_error(__VA_ARGS__);           \
      return (code);                        \
    }                                       \
  } while (0)

static inline bool ody_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---------------------------------------------------------------------------
// device helpers
// ---------------------------------------------------------------------------
__device__ __forceinline__ float ody_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <typename T> __device__ __forceinline__ float to_f32(T x);
template <> __device__ __forceinline__ float to_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ float to_f32<bf16>(bf16 x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float x) { return (bf16)x; }

// 64-bit LDS transpose read (gfx950 ds_read_b64_tr_b16).  Within each block of
// 16 lanes, lane j supplies the address of 4 consecutive 16-bit elements
// M[j][0..3]; lane i receives M[4k + i/4][i%4] for k = 0..3.  With lane j
// pointing at row (j>>2), column 4*(j&3) of a row-major tile, lane i ends up
// with 4 consecutive ROWS of column i: a 4x16 -> 16x4 transpose.
__device__ __forceinline__ bf16x4 lds_read_tr16(const bf16* p) {
  typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
  return __builtin_bit_cast(bf16x4, v);
}

__device__ __forceinline__ bf16x8 concat4(bf16x4 lo, bf16x4 hi) {
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// Exchange with the lane 32 positions away (the other half of the wavefront).
__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32, 64); }

template <typename T> struct Vec16B;  // 16-byte vector of T
template <> struct Vec16B<bf16> { typedef bf16x8 type; static constexpr int N = 8; };
template <> struct Vec16B<float> { typedef f32x4 type; static constexpr int N = 4; };
