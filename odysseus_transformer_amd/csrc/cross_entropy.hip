// Fused softmax cross-entropy over the vocabulary, forward and in-place backward: the loss the
// reference's training loop takes from flash_attn (CrossEntropyLoss(inplace_backward=True),
// train.py:8,173,212-214).  Memory-bound: the forward reads every logit once, the backward reads
// it once more and overwrites it with its gradient.  One 256-thread block per token row, 16-byte
// loads, fp32 statistics, online (max, sum) per lane and one block reduction per row.
#include <cmath>
#include "ody_common.h"

namespace {

template <typename T> struct RowIO {
  static constexpr int N = Vec16B<T>::N;
  typedef typename Vec16B<T>::type vec_t;
};

struct MaxSum { float m, s; };   // running maximum and sum of exp(x - m)

__device__ __forceinline__ MaxSum combine(MaxSum a, MaxSum b) {
  const float m = fmaxf(a.m, b.m);
  if (m == -INFINITY) return MaxSum{m, 0.f};
  return MaxSum{m, a.s * __expf(a.m - m) + b.s * __expf(b.m - m)};
}

__device__ __forceinline__ MaxSum block_combine(MaxSum v, MaxSum* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    MaxSum w{__shfl_xor(v.m, o, 64), __shfl_xor(v.s, o, 64)};
    v = combine(v, w);
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) red[wave] = v;
  __syncthreads();
  MaxSum r = red[0];
#pragma unroll
  for (int w = 1; w < 4; w++) r = combine(r, red[w]);
  return r;
}

// losses[t] = lse[t] - logits[t, label[t]] (0 for an ignored token); lse[t] = log sum_v exp(logits[t, v])
template <typename T>
__global__ __launch_bounds__(256) void ce_fwd_kernel(const T* __restrict__ logits, const int64_t* __restrict__ labels,
                                                     float* __restrict__ losses, float* __restrict__ lse_out, int V,
                                                     int64_t ld, int64_t ignore_index, bool vec_ok) {
  constexpr int N = RowIO<T>::N;
  typedef typename RowIO<T>::vec_t vec_t;
  __shared__ MaxSum red[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  const T* x = logits + (int64_t)row * ld;
  MaxSum acc{-INFINITY, 0.f};
  const int nvec = vec_ok ? V / N : 0;
  for (int vi = tid; vi < nvec; vi += 256) {
    const vec_t v = *reinterpret_cast<const vec_t*>(x + (int64_t)vi * N);
    float m = (float)v[0];
#pragma unroll
    for (int e = 1; e < N; e++) m = fmaxf(m, (float)v[e]);
    const float nm = fmaxf(acc.m, m);
    float s = acc.s * __expf(acc.m - nm);   // acc.m = -inf gives 0 * 0
    if (nm == -INFINITY) s = 0.f;
    else {
#pragma unroll
      for (int e = 0; e < N; e++) s += __expf((float)v[e] - nm);
    }
    acc = MaxSum{nm, s};
  }
  for (int c = nvec * N + tid; c < V; c += 256) acc = combine(acc, MaxSum{(float)x[c], 1.f});
  const MaxSum r = block_combine(acc, red);
  if (tid == 0) {
    const float lse = r.m + __logf(r.s);
    const int64_t lab = labels[row];
    const bool valid = lab != ignore_index && lab >= 0 && lab < V;
    lse_out[row] = lse;
    // a label outside [0, V) that is not ignore_index is a bug upstream (a vocabulary off by one, say): its loss is
    // NaN, and so is every mean or sum it enters, instead of a token silently left out
    losses[row] = valid ? lse - (float)x[lab] : (lab == ignore_index ? 0.f : __builtin_nanf(""));
  }
}

// reduced[0] = mean of the losses over the tokens that count, reduced[1] = their number.
// One block, fixed summation order: deterministic.
__global__ __launch_bounds__(1024) void ce_reduce_kernel(const float* __restrict__ losses,
                                                         const int64_t* __restrict__ labels, float* __restrict__ reduced,
                                                         int T, int V, int64_t ignore_index) {
  __shared__ float ssum[16], scnt[16];
  float s = 0.f, c = 0.f;
  for (int t = threadIdx.x; t < T; t += 1024) {
    const int64_t lab = labels[t];
    if (lab != ignore_index) s += losses[t], c += 1.f;   // a label out of range counts, with its NaN
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64), c += __shfl_xor(c, o, 64);
  if ((threadIdx.x & 63) == 0) ssum[threadIdx.x >> 6] = s, scnt[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    float ts = 0.f, tc = 0.f;
    for (int w = 0; w < 16; w++) ts += ssum[w], tc += scnt[w];
    reduced[0] = tc > 0.f ? ts / tc : 0.f;
    reduced[1] = tc;
  }
}

// In place: logits[t, v] <- (softmax(logits[t])[v] - [v == label[t]]) * g, with
// g = grad_loss[0] / reduced[1] (mean over the counted tokens) or dloss[t] (per-token gradient);
// an ignored token's row becomes 0.
template <typename T>
__global__ __launch_bounds__(256) void ce_bwd_kernel(T* __restrict__ logits, const int64_t* __restrict__ labels,
                                                     const float* __restrict__ lse, const float* __restrict__ reduced,
                                                     const float* __restrict__ grad_loss,
                                                     const float* __restrict__ dloss, int V, int64_t ld,
                                                     int64_t ignore_index, bool vec_ok) {
  constexpr int N = RowIO<T>::N;
  typedef typename RowIO<T>::vec_t vec_t;
  const int row = blockIdx.x, tid = threadIdx.x;
  T* x = logits + (int64_t)row * ld;
  const int64_t lab = labels[row];
  const bool valid = lab != ignore_index && lab >= 0 && lab < V;
  float g = 0.f;
  if (valid) g = dloss ? dloss[row] : grad_loss[0] / fmaxf(reduced[1], 1.f);
  const float l = lse[row];
  const int ilab = valid ? (int)lab : -1;
  const int nvec = vec_ok ? V / N : 0;
  for (int vi = tid; vi < nvec; vi += 256) {
    vec_t v = *reinterpret_cast<const vec_t*>(x + (int64_t)vi * N);
#pragma unroll
    for (int e = 0; e < N; e++) {
      const float p = __expf((float)v[e] - l);
      v[e] = (T)((p - (vi * N + e == ilab ? 1.f : 0.f)) * g);
    }
    *reinterpret_cast<vec_t*>(x + (int64_t)vi * N) = v;
  }
  for (int c = nvec * N + tid; c < V; c += 256) {
    const float p = __expf((float)x[c] - l);
    x[c] = (T)((p - (c == ilab ? 1.f : 0.f)) * g);
  }
}

int check(const char* who, const void* logits, const int64_t* labels, int T, int V, int64_t ld, int dtype) {
  ODY_REQUIRE(logits && labels, ODY_ERR_NULL, "%s: NULL pointer", who);
  ODY_REQUIRE(T > 0 && V > 0 && ld >= V, ODY_ERR_BAD_SHAPE, "%s: T=%d V=%d ld=%lld", who, T, V, (long long)ld);
  ODY_REQUIRE(dtype == ODY_BF16 || dtype == ODY_F32, ODY_ERR_UNSUPPORTED, "%s: dtype %d unknown", who, dtype);
  return ODY_OK;
}

// 16-byte row accesses need an aligned base and a row pitch that keeps every row aligned
bool rows_aligned(const void* p, int64_t ld, int dtype) {
  const int q = dtype == ODY_BF16 ? 8 : 4;
  return ody_aligned16(p) && ld % q == 0;
}

}  // namespace

extern "C" int ody_cross_entropy_fwd(const void* logits, const int64_t* labels, float* losses, float* lse,
                                     float* reduced, int T, int V, int64_t ld, int64_t ignore_index, int dtype,
                                     void* stream) {
  int rc = check("ody_cross_entropy_fwd", logits, labels, T, V, ld, dtype);
  if (rc) return rc;
  ODY_REQUIRE(losses && lse, ODY_ERR_NULL, "ody_cross_entropy_fwd: losses / lse is NULL");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = rows_aligned(logits, ld, dtype);
  if (dtype == ODY_BF16)
    ODY_LAUNCH("cross_entropy_fwd", st, ce_fwd_kernel<bf16>, dim3(T), dim3(256), 0, static_cast<const bf16*>(logits),
               labels, losses, lse, V, ld, ignore_index, vec);
  else
    ODY_LAUNCH("cross_entropy_fwd", st, ce_fwd_kernel<float>, dim3(T), dim3(256), 0, static_cast<const float*>(logits),
               labels, losses, lse, V, ld, ignore_index, vec);
  if ((rc = ody_check_launch("cross_entropy_fwd"))) return rc;
  if (reduced) {
    ODY_LAUNCH("cross_entropy_reduce", st, ce_reduce_kernel, dim3(1), dim3(1024), 0, losses, labels, reduced, T, V,
               ignore_index);
    rc = ody_check_launch("cross_entropy_reduce");
  }
  return rc;
}

extern "C" int ody_cross_entropy_bwd(void* logits, const int64_t* labels, const float* lse, const float* reduced,
                                     const float* grad_loss, const float* dloss, int T, int V, int64_t ld,
                                     int64_t ignore_index, int dtype, void* stream) {
  int rc = check("ody_cross_entropy_bwd", logits, labels, T, V, ld, dtype);
  if (rc) return rc;
  ODY_REQUIRE(lse != nullptr, ODY_ERR_NULL, "ody_cross_entropy_bwd: lse is NULL");
  ODY_REQUIRE(dloss != nullptr || (reduced != nullptr && grad_loss != nullptr), ODY_ERR_NULL,
              "ody_cross_entropy_bwd: pass either dloss (per token) or reduced and grad_loss (mean reduction)");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = rows_aligned(logits, ld, dtype);
  if (dtype == ODY_BF16)
    ODY_LAUNCH("cross_entropy_bwd", st, ce_bwd_kernel<bf16>, dim3(T), dim3(256), 0, static_cast<bf16*>(logits), labels,
               lse, reduced, grad_loss, dloss, V, ld, ignore_index, vec);
  else
    ODY_LAUNCH("cross_entropy_bwd", st, ce_bwd_kernel<float>, dim3(T), dim3(256), 0, static_cast<float*>(logits), labels,
               lse, reduced, grad_loss, dloss, V, ld, ignore_index, vec);
  return ody_check_launch("cross_entropy_bwd");
}
