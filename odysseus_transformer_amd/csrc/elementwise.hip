// Memory-bound kernels of the decoder layer: RMSNorm, RoPE, SwiGLU, LSE merge.
// All move 16-byte vectors per lane, keep statistics in fp32 and reduce inside a
// wavefront with lane shuffles; none of them is shaped into a matrix product.
#include <cmath>
#include <algorithm>
#include <cmath>
#include "ody_common.h"

namespace {

template <typename T> struct VecIO {
  static constexpr int N = Vec16B<T>::N;
  typedef typename Vec16B<T>::type vec_t;
  __device__ static __forceinline__ void load(const T* p, float (&f)[N]) {
    const vec_t v = *reinterpret_cast<const vec_t*>(p);
#pragma unroll
    for (int e = 0; e < N; e++) f[e] = (float)v[e];
  }
  __device__ static __forceinline__ void store(T* p, const float (&f)[N]) {
    vec_t v;
#pragma unroll
    for (int e = 0; e < N; e++) v[e] = (T)f[e];
    *reinterpret_cast<vec_t*>(p) = v;
  }
  // Streaming forms: a result that this kernel does not read again leaves without taking cache room from the
  // operands (measured on d = 4096 bf16 rows: RMSNorm forward 11.2 -> 8.3 us at 4096 rows, 94 -> 78 us at 32768), and
  // operands too large for the last-level cache to hold anyway are read past it.
  typedef unsigned raw_t __attribute__((ext_vector_type(4)));
  __device__ static __forceinline__ vec_t load_raw(const T* p, bool streaming) {
    if (streaming) return __builtin_bit_cast(vec_t, __builtin_nontemporal_load(reinterpret_cast<const raw_t*>(p)));
    return *reinterpret_cast<const vec_t*>(p);
  }
  __device__ static __forceinline__ void store_streaming(T* p, const float (&f)[N]) {
    vec_t v;
#pragma unroll
    for (int e = 0; e < N; e++) v[e] = (T)f[e];
    __builtin_nontemporal_store(__builtin_bit_cast(raw_t, v), reinterpret_cast<raw_t*>(p));
  }
};

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int s = 32; s > 0; s >>= 1) x += __shfl_xor(x, s, 64);
  return x;
}

// round-trip through the storage type (a no-op for fp32)
template <typename T> __device__ __forceinline__ float rnd(float x) { return (float)(T)x; }

// ---------------------------------------------------------------------------
// RMSNorm forward: one wavefront per row; the row is cached in registers when it
// fits (d <= 64 * N * CACHE), otherwise re-read.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_fwd_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                          T* __restrict__ y, float* __restrict__ rstd_out, int Trows,
                                                          int d, float eps) {
  constexpr int N = VecIO<T>::N, CACHE = 8;
  const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= Trows) return;
  const T* xr = x + (int64_t)row * d;
  T* yr = y + (int64_t)row * d;
  const int nvec = d / N;
  float cache[CACHE][N];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CACHE; c++) {
    const int vi = lane + 64 * c;
    if (vi < nvec) {
      VecIO<T>::load(xr + vi * N, cache[c]);
#pragma unroll
      for (int e = 0; e < N; e++) ss = fmaf(cache[c][e], cache[c][e], ss);
    }
  }
  for (int vi = lane + 64 * CACHE; vi < nvec; vi += 64) {
    float f[N];
    VecIO<T>::load(xr + vi * N, f);
#pragma unroll
    for (int e = 0; e < N; e++) ss = fmaf(f[e], f[e], ss);
  }
  ss = wave_sum(ss);
  const float rstd = rsqrtf(ss / (float)d + eps);
  if (lane == 0 && rstd_out) rstd_out[row] = rstd;
#pragma unroll
  for (int c = 0; c < CACHE; c++) {
    const int vi = lane + 64 * c;
    if (vi < nvec) {
      float wf[N], o[N];
      VecIO<T>::load(w + vi * N, wf);
#pragma unroll
      for (int e = 0; e < N; e++) o[e] = wf[e] * rnd<T>(cache[c][e] * rstd);
      VecIO<T>::store_streaming(yr + vi * N, o);
    }
  }
  for (int vi = lane + 64 * CACHE; vi < nvec; vi += 64) {
    float f[N], wf[N], o[N];
    VecIO<T>::load(xr + vi * N, f);
    VecIO<T>::load(w + vi * N, wf);
#pragma unroll
    for (int e = 0; e < N; e++) o[e] = wf[e] * rnd<T>(f[e] * rstd);
    VecIO<T>::store_streaming(yr + vi * N, o);
  }
}

// ---------------------------------------------------------------------------
// RMSNorm backward.  A block owns a contiguous range of rows; for each row its
// 4 wavefronts compute c = mean(g * xhat) (g = dy * w) and write
// dx = rstd * (g - xhat * c); every lane also accumulates dy * xhat for its own
// columns, written at the end as one row of the fp32 partial-sum matrix.
// ---------------------------------------------------------------------------
constexpr int RMS_BWD_MAXK = 4;  // column vectors per lane: d <= 256 * N * MAXK

// MAXK: column vectors per lane this instance is built for (d <= 256 * N * MAXK).  The raw vectors of the next
// row are fetched before the current row's sum is reduced, so that a block always has a row of loads in flight.
// EXACT: d == 256 * N * MAXK, every lane owns MAXK vectors; ADD: dx_add is there.  Both are compile-time so that the
// loads sit in straight-line code: behind a run-time test the compiler no longer counts the loads in flight and
// waits for all of them before the first use, which serialises the prefetch (measured on 4096 rows of 4096 bf16:
// 24.8 us with the tests, 17.6 without).
// STREAM: x, dy and dx_add are read past the caches (for operands that the 256 MB last-level cache cannot hold
// between their producer and this kernel; measured at 32768 rows of 4096 bf16: 155 -> 131 us, at 4096 rows, where they
// can: 17.7 -> 20.5 us).  dx always leaves by streaming stores.
template <typename T, int MAXK, bool STREAM, bool EXACT, bool ADD>
__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                          const float* __restrict__ rstd, const T* __restrict__ dy,
                                                          T* __restrict__ dx, float* __restrict__ dw_partial,
                                                          int Trows, int d, int rows_per_block,
                                                          const T* __restrict__ dx_add) {
  constexpr int N = VecIO<T>::N;
  typedef typename VecIO<T>::vec_t vec_t;
  __shared__ float red[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nvec = d / N;
  const int r0 = blockIdx.x * rows_per_block, r1 = min(Trows, r0 + rows_per_block);
  auto owns = [&](int k) { return EXACT || tid + 256 * k < nvec; };
  float wf[MAXK][N], acc[MAXK][N];
#pragma unroll
  for (int k = 0; k < MAXK; k++) {
#pragma unroll
    for (int e = 0; e < N; e++) acc[k][e] = 0.f, wf[k][e] = 0.f;
    if (owns(k)) VecIO<T>::load(w + (tid + 256 * k) * N, wf[k]);
  }
  vec_t xr[MAXK], dyr[MAXK], ar[MAXK];   // raw vectors of the row in hand
  auto fetch = [&](int row, vec_t (&xv)[MAXK], vec_t (&dv)[MAXK], vec_t (&av)[MAXK]) {
#pragma unroll
    for (int k = 0; k < MAXK; k++) {
      const int64_t at = (int64_t)row * d + (tid + 256 * k) * N;
      if (owns(k)) {
        xv[k] = VecIO<T>::load_raw(x + at, STREAM);
        dv[k] = VecIO<T>::load_raw(dy + at, STREAM);
        if (ADD) av[k] = VecIO<T>::load_raw(dx_add + at, STREAM);
      }
    }
  };
  if (r0 < r1) fetch(r0, xr, dyr, ar);
  for (int row = r0; row < r1; row++) {
    vec_t xn[MAXK], dyn[MAXK], an[MAXK];
    if (row + 1 < r1) fetch(row + 1, xn, dyn, an);
    const float rs = rstd[row];
    float xh[MAXK][N], gv[MAXK][N];
    float part = 0.f;
#pragma unroll
    for (int k = 0; k < MAXK; k++) {
      if (owns(k)) {
#pragma unroll
        for (int e = 0; e < N; e++) {
          const float dyv = (float)dyr[k][e];
          xh[k][e] = (float)xr[k][e] * rs;
          gv[k][e] = dyv * wf[k][e];
          part = fmaf(gv[k][e], xh[k][e], part);
          acc[k][e] = fmaf(dyv, xh[k][e], acc[k][e]);
        }
      }
    }
    part = wave_sum(part);
    const int pb = (row - r0) & 1;  // alternate slots so that one barrier per row suffices
    if (lane == 0) red[pb][wave] = part;
    __syncthreads();
    const float c = (red[pb][0] + red[pb][1] + red[pb][2] + red[pb][3]) / (float)d;
#pragma unroll
    for (int k = 0; k < MAXK; k++) {
      if (owns(k)) {
        float o[N];
#pragma unroll
        for (int e = 0; e < N; e++) {
          const float add = ADD ? (float)ar[k][e] : 0.f;   // gradient arriving over the residual path
          o[e] = add + rs * (gv[k][e] - xh[k][e] * c);
        }
        VecIO<T>::store_streaming(dx + (int64_t)row * d + (tid + 256 * k) * N, o);
      }
    }
    if (row + 1 < r1) {
#pragma unroll
      for (int k = 0; k < MAXK; k++) xr[k] = xn[k], dyr[k] = dyn[k], ar[k] = an[k];
    }
  }
#pragma unroll
  for (int k = 0; k < MAXK; k++) {
    if (owns(k)) {
      float* dst = dw_partial + (int64_t)blockIdx.x * d + (tid + 256 * k) * N;
#pragma unroll
      for (int h = 0; h < N / 4; h++)
        *reinterpret_cast<f32x4*>(dst + 4 * h) = f32x4{acc[k][4 * h], acc[k][4 * h + 1], acc[k][4 * h + 2], acc[k][4 * h + 3]};
    }
  }
}

template <typename T, int K, bool STREAM, bool EXACT>
void launch_rmsnorm_bwd_k(hipStream_t st, int nblocks, const void* x, const void* w, const float* rstd, const void* dy,
                          void* dx, float* dw_partial, int T_, int d, int rpb, const void* dx_add) {
  if (dx_add)
    ODY_LAUNCH("rmsnorm_bwd", st, (rmsnorm_bwd_kernel<T, K, STREAM, EXACT, true>), dim3(nblocks), dim3(256), 0, (const T*)x,
               (const T*)w, rstd, (const T*)dy, (T*)dx, dw_partial, T_, d, rpb, (const T*)dx_add);
  else
    ODY_LAUNCH("rmsnorm_bwd", st, (rmsnorm_bwd_kernel<T, K, STREAM, EXACT, false>), dim3(nblocks), dim3(256), 0, (const T*)x,
               (const T*)w, rstd, (const T*)dy, (T*)dx, dw_partial, T_, d, rpb, (const T*)nullptr);
}

template <typename T>
void launch_rmsnorm_bwd(hipStream_t st, int nblocks, const void* x, const void* w, const float* rstd, const void* dy,
                        void* dx, float* dw_partial, int T_, int d, int rpb, const void* dx_add) {
  const int nvec = d / VecIO<T>::N;
  // operands and result together beyond what the last-level cache holds: read them past it
  const bool stream = (size_t)(dx_add ? 4 : 3) * T_ * d * sizeof(T) > ((size_t)192 << 20);
#define ODY_RMS_BWD(K)                                                                                              \
  do {                                                                                                              \
    if (nvec != 256 * K) launch_rmsnorm_bwd_k<T, K, false, false>(st, nblocks, x, w, rstd, dy, dx, dw_partial, T_, d, rpb, dx_add); \
    else if (stream) launch_rmsnorm_bwd_k<T, K, true, true>(st, nblocks, x, w, rstd, dy, dx, dw_partial, T_, d, rpb, dx_add);      \
    else launch_rmsnorm_bwd_k<T, K, false, true>(st, nblocks, x, w, rstd, dy, dx, dw_partial, T_, d, rpb, dx_add);                 \
  } while (0)
  if (nvec <= 256) ODY_RMS_BWD(1);
  else if (nvec <= 512) ODY_RMS_BWD(2);
  else ODY_RMS_BWD(4);
#undef ODY_RMS_BWD
}

// out[c] = sum_r partial[r][c], d a multiple of 4.  A block owns 64 columns (256-byte row pieces, a 16-byte load per
// thread) and splits the rows over 16 thread groups that keep 4 loads in flight; d / 64 blocks share the reading.
template <typename T>
__global__ __launch_bounds__(256) void colsum_kernel(const float* __restrict__ partial, T* __restrict__ out, int n,
                                                     int d) {
  __shared__ f32x4 red[16][17];
  const int cl = threadIdx.x & 15, rg = threadIdx.x >> 4, c4 = blockIdx.x * 16 + cl, d4 = d / 4;   // columns 4 c4 .. + 3
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
  if (c4 < d4) {
    const f32x4* src = reinterpret_cast<const f32x4*>(partial) + c4;
    int r = rg;
    for (; r + 48 < n; r += 64) {
      const f32x4 a = src[(int64_t)r * d4], b = src[(int64_t)(r + 16) * d4], c = src[(int64_t)(r + 32) * d4],
                  e = src[(int64_t)(r + 48) * d4];
      s += (a + b) + (c + e);
    }
    for (; r < n; r += 16) s += src[(int64_t)r * d4];
  }
  red[rg][cl] = s;
  __syncthreads();
  if (rg == 0 && c4 < d4) {
#pragma unroll
    for (int k = 1; k < 16; k++) s += red[k][cl];
#pragma unroll
    for (int e = 0; e < 4; e++) out[4 * c4 + e] = (T)s[e];
  }
}

// ---------------------------------------------------------------------------
// RoPE, half-rotation convention, in place.  A thread owns N frequency indices
// j..j+N-1 of one (batch, position), evaluates cos/sin once and walks over the
// heads: x[j] <- x[j]*c - x[j+D/2]*s ; x[j+D/2] <- x[j+D/2]*c + x[j]*s
// (inverse: s -> -s).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void rope_kernel(T* __restrict__ x, const int64_t* __restrict__ pos_ids,
                                                   const float* __restrict__ inv_freq, int B, int L, int n_rot, int D,
                                                   int64_t sb, int64_t sl, int64_t sh, float log2_base, int inverse) {
  constexpr int N = VecIO<T>::N;
  const int half = D / 2, vph = half / N;  // vectors per half row
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)B * L * vph) return;
  const int jv = idx % vph;
  const int l = (idx / vph) % L;
  const int b = idx / ((int64_t)vph * L);
  const float pos = pos_ids ? (float)pos_ids[(int64_t)b * L + l] : (float)l;
  float cs[N], sn[N];
#pragma unroll
  for (int e = 0; e < N; e++) {
    const int j = jv * N + e;
    const float f = inv_freq ? inv_freq[j] : exp2f(-(2.0f * j / D) * log2_base);
    const float th = pos * f;
    // cos/sin are rounded to the storage type before use, as the caller of the
    // replaced routine does (cos.to(dtype), sin.to(dtype))
    cs[e] = rnd<T>(cosf(th));
    sn[e] = rnd<T>(sinf(th));
    if (inverse) sn[e] = -sn[e];
  }
  T* base = x + b * sb + (int64_t)l * sl + jv * N;
  for (int h = 0; h < n_rot; h++) {
    T* p1 = base + h * sh;
    T* p2 = p1 + half;
    float a[N], c[N], o1[N], o2[N];
    VecIO<T>::load(p1, a);
    VecIO<T>::load(p2, c);
#pragma unroll
    for (int e = 0; e < N; e++) {
      o1[e] = a[e] * cs[e] - c[e] * sn[e];
      o2[e] = c[e] * cs[e] + a[e] * sn[e];
    }
    VecIO<T>::store(p1, o1);
    VecIO<T>::store(p2, o2);
  }
}

// cos / sin of every (row, frequency) once, rounded to bf16 as rope_kernel rounds them: table[row][2 j] = cos,
// table[row][2 j + 1] = sin of pos[row] * inv_freq[j], j < D / 2.  The fused QKV projection and the attention
// backward read it instead of evaluating sincos in their epilogues.
__global__ __launch_bounds__(256) void rope_table_kernel(const int64_t* __restrict__ pos_ids,
                                                         const float* __restrict__ inv_freq, int64_t rows, int D,
                                                         float log2_base, bf16* __restrict__ table) {
  const int half = D / 2;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * half) return;
  const int j = idx % half;
  const int64_t row = idx / half;
  const float pos = pos_ids ? (float)pos_ids[row] : (float)row;
  const float f = inv_freq ? inv_freq[j] : exp2f(-(2.0f * j / D) * log2_base);
  const float th = pos * f;
  typedef __attribute__((__vector_size__(2 * sizeof(bf16)))) bf16 bf16x2;
  *reinterpret_cast<bf16x2*>(table + row * D + 2 * j) = bf16x2{(bf16)cosf(th), (bf16)sinf(th)};
}

// In-place rotation of the first n_rot heads of x (rows, heads, D) bf16 with the table above; 8 frequencies per thread.
__global__ __launch_bounds__(256) void rope_from_table_kernel(bf16* __restrict__ x, const bf16* __restrict__ table,
                                                              int64_t rows, int n_rot, int D, int64_t s_row, int64_t s_h,
                                                              int inverse) {
  const int half = D / 2, vph = half / 8;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * vph) return;
  const int jv = idx % vph;
  const int64_t row = idx / vph;
  const bf16x8 t0 = *reinterpret_cast<const bf16x8*>(table + row * D + 16 * jv);
  const bf16x8 t1 = *reinterpret_cast<const bf16x8*>(table + row * D + 16 * jv + 8);
  float cs[8], sn[8];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    cs[e] = (float)t0[2 * e], sn[e] = (float)t0[2 * e + 1];
    cs[4 + e] = (float)t1[2 * e], sn[4 + e] = (float)t1[2 * e + 1];
  }
  if (inverse) {
#pragma unroll
    for (int e = 0; e < 8; e++) sn[e] = -sn[e];
  }
  bf16* base = x + row * s_row + jv * 8;
  for (int h = 0; h < n_rot; h++) {
    bf16* p1 = base + h * s_h;
    bf16* p2 = p1 + half;
    const bf16x8 a = *reinterpret_cast<const bf16x8*>(p1), c = *reinterpret_cast<const bf16x8*>(p2);
    bf16x8 o1, o2;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      o1[e] = (bf16)((float)a[e] * cs[e] - (float)c[e] * sn[e]);
      o2[e] = (bf16)((float)c[e] * cs[e] + (float)a[e] * sn[e]);
    }
    *reinterpret_cast<bf16x8*>(p1) = o1;
    *reinterpret_cast<bf16x8*>(p2) = o2;
  }
}

// ---------------------------------------------------------------------------
// SwiGLU
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const T* __restrict__ gu, T* __restrict__ h, int Trows, int I,
                                                         int64_t ld_gu, int64_t ld_h) {
  constexpr int N = VecIO<T>::N;
  const int vpr = I / N;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)Trows * vpr) return;
  const int jv = idx % vpr;
  const int64_t t = idx / vpr;
  float a1[N], a3[N], o[N];
  VecIO<T>::load(gu + t * ld_gu + jv * N, a1);
  VecIO<T>::load(gu + t * ld_gu + I + jv * N, a3);
#pragma unroll
  for (int e = 0; e < N; e++) o[e] = a1[e] / (1.f + __expf(-a1[e])) * a3[e];
  VecIO<T>::store(h + t * ld_h + jv * N, o);   // (a streaming store was measured 2-3 % slower here)
}

template <typename T>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T* __restrict__ gu, const T* __restrict__ dh,
                                                         T* __restrict__ dgu, int Trows, int I, int64_t ld_gu,
                                                         int64_t ld_dh, int64_t ld_dgu) {
  constexpr int N = VecIO<T>::N;
  const int vpr = I / N;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)Trows * vpr) return;
  const int jv = idx % vpr;
  const int64_t t = idx / vpr;
  float a1[N], a3[N], g[N], d1[N], d3[N];
  VecIO<T>::load(gu + t * ld_gu + jv * N, a1);
  VecIO<T>::load(gu + t * ld_gu + I + jv * N, a3);
  VecIO<T>::load(dh + t * ld_dh + jv * N, g);
#pragma unroll
  for (int e = 0; e < N; e++) {
    const float sig = 1.f / (1.f + __expf(-a1[e]));
    d1[e] = g[e] * a3[e] * sig * (1.f + a1[e] * (1.f - sig));
    d3[e] = g[e] * a1[e] * sig;
  }
  VecIO<T>::store_streaming(dgu + t * ld_dgu + jv * N, d1);
  VecIO<T>::store_streaming(dgu + t * ld_dgu + I + jv * N, d3);
}

// ---------------------------------------------------------------------------
// LSE merge: 4 head-dim elements per lane, D/4 lanes per (b, l, h) row.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void lse_merge_kernel(float* __restrict__ out_acc, float* __restrict__ lse_acc,
                                                        const T* __restrict__ out_blk,
                                                        const float* __restrict__ lse_blk, int B, int L, int H, int D,
                                                        int64_t sb, int64_t sl, int64_t sh) {
  const int lpr = D / 4;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)B * L * H * lpr) return;
  const int sub = idx % lpr;
  const int64_t row = idx / lpr;  // (b, l, h) order
  const int h = row % H;
  const int l = (row / H) % L;
  const int b = row / ((int64_t)H * L);
  const int64_t li = ((int64_t)b * H + h) * L + l;
  const float a = lse_acc[li], c = lse_blk[li];
  const float mx = fmaxf(a, c);
  float nw, wa, wb;
  if (mx == -INFINITY) {
    nw = -INFINITY, wa = 0.f, wb = 0.f;
  } else {
    nw = mx + logf(expf(a - mx) + expf(c - mx));
    wa = expf(a - nw), wb = expf(c - nw);
  }
  float* oa = out_acc + row * D + sub * 4;
  const T* ob = out_blk + b * sb + (int64_t)l * sl + h * sh + sub * 4;
  f32x4 va = *reinterpret_cast<const f32x4*>(oa);
  float vb[4];
  if constexpr (sizeof(T) == 2) {
    const bf16x4 t = *reinterpret_cast<const bf16x4*>(ob);
#pragma unroll
    for (int e = 0; e < 4; e++) vb[e] = (float)t[e];
  } else {
    const f32x4 t = *reinterpret_cast<const f32x4*>(ob);
#pragma unroll
    for (int e = 0; e < 4; e++) vb[e] = t[e];
  }
#pragma unroll
  for (int e = 0; e < 4; e++) va[e] = va[e] * wa + vb[e] * wb;
  *reinterpret_cast<f32x4*>(oa) = va;
  // every lane of this row sits in one wavefront and has read lse_acc above
  if (sub == 0) lse_acc[li] = nw;
}

inline unsigned blocks_for(int64_t n) { return (unsigned)((n + 255) / 256); }

template <typename T> constexpr int vecn() { return Vec16B<T>::N; }

}  // namespace

#define ODY_BY_DTYPE(dtype, EXPR_BF16, EXPR_F32)                         \
  if ((dtype) == ODY_BF16) { EXPR_BF16; }                                \
  else if ((dtype) == ODY_F32) { EXPR_F32; }                             \
  else { ody_set_error("dtype %d unknown", (dtype)); return ODY_ERR_UNSUPPORTED; }

extern "C" int ody_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd, int T, int d, float eps, int dtype,
                               void* stream) {
  ODY_REQUIRE(x && w && y, ODY_ERR_NULL, "ody_rmsnorm_fwd: NULL pointer");
  ODY_REQUIRE(T > 0 && d > 0, ODY_ERR_BAD_SHAPE, "ody_rmsnorm_fwd: T=%d d=%d", T, d);
  const int n = dtype == ODY_BF16 ? 8 : 4;
  ODY_REQUIRE(d % n == 0, ODY_ERR_UNSUPPORTED, "ody_rmsnorm_fwd: d=%d must be a multiple of %d", d, n);
  ODY_REQUIRE(ody_aligned16(x) && ody_aligned16(w) && ody_aligned16(y), ODY_ERR_MISALIGNED,
              "ody_rmsnorm_fwd: pointers must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  dim3 grid((T + 3) / 4);
  ODY_BY_DTYPE(dtype,
               ODY_LAUNCH("rmsnorm_fwd", st, rmsnorm_fwd_kernel<bf16>, grid, dim3(256), 0, (const bf16*)x, (const bf16*)w,
                                  (bf16*)y, rstd, T, d, eps),
               ODY_LAUNCH("rmsnorm_fwd", st, rmsnorm_fwd_kernel<float>, grid, dim3(256), 0, (const float*)x, (const float*)w,
                                  (float*)y, rstd, T, d, eps));
  return ody_check_launch("rmsnorm_fwd");
}

// one block per compute unit: more blocks only add partial sums to write and read back
extern "C" int ody_rmsnorm_bwd_partials(int T) { return T <= 0 ? 0 : (T < 256 ? T : 256); }

extern "C" int ody_rmsnorm_bwd(const void* x, const void* w, const float* rstd, const void* dy, const void* dx_add,
                               void* dx, float* dw_partial, void* dw, int T, int d, int dtype, void* stream) {
  ODY_REQUIRE(x && w && rstd && dy && dx && dw_partial, ODY_ERR_NULL, "ody_rmsnorm_bwd: NULL pointer");
  ODY_REQUIRE(T > 0 && d > 0, ODY_ERR_BAD_SHAPE, "ody_rmsnorm_bwd: T=%d d=%d", T, d);
  const int n = dtype == ODY_BF16 ? 8 : 4;
  ODY_REQUIRE(d % n == 0 && d <= 256 * n * RMS_BWD_MAXK, ODY_ERR_UNSUPPORTED,
              "ody_rmsnorm_bwd: d=%d must be a multiple of %d and at most %d", d, n, 256 * n * RMS_BWD_MAXK);
  ODY_REQUIRE(ody_aligned16(x) && ody_aligned16(w) && ody_aligned16(dy) && ody_aligned16(dx) && ody_aligned16(dx_add) &&
                  ody_aligned16(dw_partial),
              ODY_ERR_MISALIGNED, "ody_rmsnorm_bwd: pointers must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int nparts = ody_rmsnorm_bwd_partials(T);
  const int rpb = (T + nparts - 1) / nparts;
  const int nblocks = (T + rpb - 1) / rpb;  // <= nparts; rows of dw_partial beyond nblocks are not written
  ODY_BY_DTYPE(dtype, launch_rmsnorm_bwd<bf16>(st, nblocks, x, w, rstd, dy, dx, dw_partial, T, d, rpb, dx_add),
               launch_rmsnorm_bwd<float>(st, nblocks, x, w, rstd, dy, dx, dw_partial, T, d, rpb, dx_add));
  int rc = ody_check_launch("rmsnorm_bwd");
  if (rc || !dw) return rc;
  ODY_BY_DTYPE(dtype,
               ODY_LAUNCH("colsum", st, colsum_kernel<bf16>, dim3((d + 63) / 64), dim3(256), 0, dw_partial, (bf16*)dw,
                                  nblocks, d),
               ODY_LAUNCH("colsum", st, colsum_kernel<float>, dim3((d + 63) / 64), dim3(256), 0, dw_partial,
                                  (float*)dw, nblocks, d));
  return ody_check_launch("rmsnorm_bwd_colsum");
}

extern "C" int ody_rope(void* x, const int64_t* position_ids, const float* inv_freq, int B, int L, int n_rot, int D,
                        int64_t sx_b, int64_t sx_l, int64_t sx_h, float base, int inverse, int dtype, void* stream) {
  ODY_REQUIRE(x, ODY_ERR_NULL, "ody_rope: x is NULL");
  ODY_REQUIRE(B > 0 && L > 0 && n_rot >= 0 && D > 0, ODY_ERR_BAD_SHAPE, "ody_rope: B=%d L=%d n_rot=%d D=%d", B, L,
              n_rot, D);
  const int n = dtype == ODY_BF16 ? 8 : 4;
  ODY_REQUIRE(D % (2 * n) == 0, ODY_ERR_UNSUPPORTED, "ody_rope: D=%d must be a multiple of %d", D, 2 * n);
  ODY_REQUIRE(ody_aligned16(x) && sx_b % n == 0 && sx_l % n == 0 && sx_h % n == 0, ODY_ERR_MISALIGNED,
              "ody_rope: x needs a 16-byte aligned pointer and strides that are multiples of %d", n);
  ODY_REQUIRE(inv_freq || base > 0.f, ODY_ERR_BAD_SHAPE, "ody_rope: base must be positive");
  if (n_rot == 0) return ODY_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t total = (int64_t)B * L * (D / 2 / n);
  const float l2b = inv_freq ? 0.f : log2f(base);
  ODY_BY_DTYPE(dtype,
               ODY_LAUNCH("rope", st, rope_kernel<bf16>, dim3(blocks_for(total)), dim3(256), 0, (bf16*)x, position_ids,
                                  inv_freq, B, L, n_rot, D, sx_b, sx_l, sx_h, l2b, inverse),
               ODY_LAUNCH("rope", st, rope_kernel<float>, dim3(blocks_for(total)), dim3(256), 0, (float*)x,
                                  position_ids, inv_freq, B, L, n_rot, D, sx_b, sx_l, sx_h, l2b, inverse));
  return ody_check_launch("rope");
}

extern "C" int ody_rope_table(const int64_t* position_ids, const float* inv_freq, int64_t rows, int D, float base,
                              void* table, void* stream) {
  ODY_REQUIRE(table, ODY_ERR_NULL, "ody_rope_table: table is NULL");
  ODY_REQUIRE(rows > 0 && D > 0 && D % 16 == 0, ODY_ERR_BAD_SHAPE, "ody_rope_table: rows=%lld D=%d (a multiple of 16)",
              (long long)rows, D);
  ODY_REQUIRE(ody_aligned16(table), ODY_ERR_MISALIGNED, "ody_rope_table: table must be 16-byte aligned");
  ODY_REQUIRE(inv_freq || base > 0.f, ODY_ERR_BAD_SHAPE, "ody_rope_table: base must be positive");
  hipStream_t st = static_cast<hipStream_t>(stream);
  ODY_LAUNCH("rope_table", st, rope_table_kernel, dim3(blocks_for(rows * (D / 2))), dim3(256), 0, position_ids, inv_freq,
             rows, D, inv_freq ? 0.f : log2f(base), static_cast<bf16*>(table));
  return ody_check_launch("rope_table");
}

// used by ody_linear_rope when the product does not take the fused kernel
int ody_launch_rope_from_table(void* x, const void* table, int64_t rows, int n_rot, int D, int64_t s_row, int64_t s_h,
                               int inverse, hipStream_t st) {
  if (n_rot == 0) return ODY_OK;
  ODY_LAUNCH("rope_from_table", st, rope_from_table_kernel, dim3(blocks_for(rows * (D / 16))), dim3(256), 0,
             static_cast<bf16*>(x), static_cast<const bf16*>(table), rows, n_rot, D, s_row, s_h, inverse);
  return ody_check_launch("rope_from_table");
}

namespace {
__global__ __launch_bounds__(256) void cast_from_f32_kernel(const float* __restrict__ src, bf16* __restrict__ dst,
                                                            int64_t n8) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n8) return;
  const f32x4 a = *reinterpret_cast<const f32x4*>(src + idx * 8), b = *reinterpret_cast<const f32x4*>(src + idx * 8 + 4);
  bf16x8 w;
#pragma unroll
  for (int e = 0; e < 4; e++) w[e] = (bf16)a[e], w[4 + e] = (bf16)b[e];
  *reinterpret_cast<bf16x8*>(dst + idx * 8) = w;
}
}  // namespace

extern "C" int ody_cast_from_f32(const float* src, void* dst, int64_t n, int dtype, void* stream) {
  ODY_REQUIRE(src && dst, ODY_ERR_NULL, "ody_cast_from_f32: NULL pointer");
  ODY_REQUIRE(n > 0 && n % 8 == 0, ODY_ERR_BAD_SHAPE, "ody_cast_from_f32: n=%lld must be a positive multiple of 8", (long long)n);
  ODY_REQUIRE(ody_aligned16(src) && ody_aligned16(dst), ODY_ERR_MISALIGNED, "ody_cast_from_f32: 16-byte alignment required");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == ODY_F32) {
    if (static_cast<const void*>(src) == dst) return ODY_OK;
    hipError_t e = hipMemcpyAsync(dst, src, (size_t)n * sizeof(float), hipMemcpyDeviceToDevice, st);
    ODY_REQUIRE(e == hipSuccess, ODY_ERR_LAUNCH, "ody_cast_from_f32: copy failed: %s", hipGetErrorString(e));
    return ODY_OK;
  }
  ODY_REQUIRE(dtype == ODY_BF16, ODY_ERR_UNSUPPORTED, "ody_cast_from_f32: dtype %d unknown", dtype);
  ODY_LAUNCH("cast_from_f32", st, cast_from_f32_kernel, dim3(blocks_for(n / 8)), dim3(256), 0, src, static_cast<bf16*>(dst),
             n / 8);
  return ody_check_launch("cast_from_f32");
}

extern "C" int ody_swiglu_fwd(const void* gate_up, void* h, int T, int I, int64_t ld_gu, int64_t ld_h, int dtype,
                              void* stream) {
  ODY_REQUIRE(gate_up && h, ODY_ERR_NULL, "ody_swiglu_fwd: NULL pointer");
  ODY_REQUIRE(T > 0 && I > 0 && ld_gu >= 2 * (int64_t)I && ld_h >= I, ODY_ERR_BAD_SHAPE,
              "ody_swiglu_fwd: T=%d I=%d ld_gu=%lld ld_h=%lld", T, I, (long long)ld_gu, (long long)ld_h);
  const int n = dtype == ODY_BF16 ? 8 : 4;
  ODY_REQUIRE(I % n == 0, ODY_ERR_UNSUPPORTED, "ody_swiglu_fwd: I=%d must be a multiple of %d", I, n);
  ODY_REQUIRE(ody_aligned16(gate_up) && ody_aligned16(h) && ld_gu % n == 0 && ld_h % n == 0, ODY_ERR_MISALIGNED,
              "ody_swiglu_fwd: 16-byte alignment of pointers and row strides required");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t total = (int64_t)T * (I / n);
  ODY_BY_DTYPE(dtype,
               ODY_LAUNCH("swiglu_fwd", st, swiglu_fwd_kernel<bf16>, dim3(blocks_for(total)), dim3(256), 0,
                                  (const bf16*)gate_up, (bf16*)h, T, I, ld_gu, ld_h),
               ODY_LAUNCH("swiglu_fwd", st, swiglu_fwd_kernel<float>, dim3(blocks_for(total)), dim3(256), 0,
                                  (const float*)gate_up, (float*)h, T, I, ld_gu, ld_h));
  return ody_check_launch("swiglu_fwd");
}

extern "C" int ody_swiglu_bwd(const void* gate_up, const void* dh, void* d_gate_up, int T, int I, int64_t ld_gu,
                              int64_t ld_dh, int64_t ld_dgu, int dtype, void* stream) {
  ODY_REQUIRE(gate_up && dh && d_gate_up, ODY_ERR_NULL, "ody_swiglu_bwd: NULL pointer");
  ODY_REQUIRE(T > 0 && I > 0 && ld_gu >= 2 * (int64_t)I && ld_dh >= I && ld_dgu >= 2 * (int64_t)I, ODY_ERR_BAD_SHAPE,
              "ody_swiglu_bwd: bad sizes T=%d I=%d", T, I);
  const int n = dtype == ODY_BF16 ? 8 : 4;
  ODY_REQUIRE(I % n == 0, ODY_ERR_UNSUPPORTED, "ody_swiglu_bwd: I=%d must be a multiple of %d", I, n);
  ODY_REQUIRE(ody_aligned16(gate_up) && ody_aligned16(dh) && ody_aligned16(d_gate_up) && ld_gu % n == 0 &&
                  ld_dh % n == 0 && ld_dgu % n == 0,
              ODY_ERR_MISALIGNED, "ody_swiglu_bwd: 16-byte alignment of pointers and row strides required");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t total = (int64_t)T * (I / n);
  ODY_BY_DTYPE(dtype,
               ODY_LAUNCH("swiglu_bwd", st, swiglu_bwd_kernel<bf16>, dim3(blocks_for(total)), dim3(256), 0,
                                  (const bf16*)gate_up, (const bf16*)dh, (bf16*)d_gate_up, T, I, ld_gu, ld_dh, ld_dgu),
               ODY_LAUNCH("swiglu_bwd", st, swiglu_bwd_kernel<float>, dim3(blocks_for(total)), dim3(256), 0,
                                  (const float*)gate_up, (const float*)dh, (float*)d_gate_up, T, I, ld_gu, ld_dh,
                                  ld_dgu));
  return ody_check_launch("swiglu_bwd");
}

extern "C" int ody_lse_merge(float* out_acc, float* lse_acc, const void* out_blk, const float* lse_blk, int B, int L,
                             int H, int D, int64_t sb_b, int64_t sb_l, int64_t sb_h, int dtype, void* stream) {
  ODY_REQUIRE(out_acc && lse_acc && out_blk && lse_blk, ODY_ERR_NULL, "ody_lse_merge: NULL pointer");
  ODY_REQUIRE(B > 0 && L > 0 && H > 0 && D > 0, ODY_ERR_BAD_SHAPE, "ody_lse_merge: B=%d L=%d H=%d D=%d", B, L, H, D);
  ODY_REQUIRE(D % 4 == 0 && D <= 256 && (64 % (D / 4) == 0), ODY_ERR_UNSUPPORTED,
              "ody_lse_merge: D=%d must be 4 times a power of two, at most 256", D);
  ODY_REQUIRE(ody_aligned16(out_acc) && ody_aligned16(out_blk) && sb_b % 4 == 0 && sb_l % 4 == 0 && sb_h % 4 == 0,
              ODY_ERR_MISALIGNED, "ody_lse_merge: alignment");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t total = (int64_t)B * L * H * (D / 4);
  ODY_BY_DTYPE(dtype,
               ODY_LAUNCH("lse_merge", st, lse_merge_kernel<bf16>, dim3(blocks_for(total)), dim3(256), 0, out_acc, lse_acc,
                                  (const bf16*)out_blk, lse_blk, B, L, H, D, sb_b, sb_l, sb_h),
               ODY_LAUNCH("lse_merge", st, lse_merge_kernel<float>, dim3(blocks_for(total)), dim3(256), 0, out_acc, lse_acc,
                                  (const float*)out_blk, lse_blk, B, L, H, D, sb_b, sb_l, sb_h));
  return ody_check_launch("lse_merge");
}

// ---------------------------------------------------------------------------
// AdamW, one pass: torch.optim.AdamW's update (train.py:170,216 of the reference) on one tensor.  Memory-bound:
// parameter, gradient and both moments are read once, parameter and moments written once (14 bytes per bf16
// parameter); the arithmetic is fp32 whatever the storage type, with one rounding per stored value.
//   p *= 1 - lr * wd;  m = b1 m + (1 - b1) g;  v = b2 v + (1 - b2) g^2;  p -= (lr / bc1) * m / (sqrt(v) / sqrt(bc2) + eps)
// ---------------------------------------------------------------------------
namespace {
template <typename T>
__global__ __launch_bounds__(256) void adamw_kernel(T* __restrict__ p, const T* __restrict__ g, T* __restrict__ m,
                                                    T* __restrict__ v, int64_t n, float decay, float b1, float b2,
                                                    float step_size, float inv_sqrt_bc2, float eps) {
  constexpr int N = VecIO<T>::N;
  const int64_t nv = n / N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nv; i += (int64_t)gridDim.x * 256) {
    float pf[N], gf[N], mf[N], vf[N];
    VecIO<T>::load(p + i * N, pf);
    VecIO<T>::load(g + i * N, gf);
    VecIO<T>::load(m + i * N, mf);
    VecIO<T>::load(v + i * N, vf);
#pragma unroll
    for (int e = 0; e < N; e++) {
      mf[e] = b1 * mf[e] + (1.f - b1) * gf[e];
      vf[e] = b2 * vf[e] + (1.f - b2) * gf[e] * gf[e];
      pf[e] = pf[e] * decay - step_size * mf[e] / (sqrtf(vf[e]) * inv_sqrt_bc2 + eps);
    }
    VecIO<T>::store(p + i * N, pf);
    VecIO<T>::store(m + i * N, mf);
    VecIO<T>::store(v + i * N, vf);
  }
  // the tail that does not fill a 16-byte vector
  if (blockIdx.x == 0 && threadIdx.x < n - nv * N) {
    const int64_t i = nv * N + threadIdx.x;
    const float gf = (float)g[i];
    const float mf = b1 * (float)m[i] + (1.f - b1) * gf;
    const float vf = b2 * (float)v[i] + (1.f - b2) * gf * gf;
    p[i] = (T)((float)p[i] * decay - step_size * mf / (sqrtf(vf) * inv_sqrt_bc2 + eps));
    m[i] = (T)mf;
    v[i] = (T)vf;
  }
}
}  // namespace

extern "C" int ody_adamw(void* param, const void* grad, void* exp_avg, void* exp_avg_sq, int64_t n, float lr, float beta1,
                         float beta2, float eps, float weight_decay, int64_t step, int dtype, void* stream) {
  ODY_REQUIRE(param && grad && exp_avg && exp_avg_sq, ODY_ERR_NULL, "ody_adamw: NULL pointer");
  ODY_REQUIRE(n > 0 && step >= 1, ODY_ERR_BAD_SHAPE, "ody_adamw: n=%lld step=%lld", (long long)n, (long long)step);
  ODY_REQUIRE(beta1 >= 0.f && beta1 < 1.f && beta2 >= 0.f && beta2 < 1.f && eps >= 0.f, ODY_ERR_BAD_SHAPE,
              "ody_adamw: betas (%g, %g) in [0, 1), eps %g >= 0", beta1, beta2, eps);
  ODY_REQUIRE(ody_aligned16(param) && ody_aligned16(grad) && ody_aligned16(exp_avg) && ody_aligned16(exp_avg_sq),
              ODY_ERR_MISALIGNED, "ody_adamw: pointers must be 16-byte aligned");
  const double bc1 = 1.0 - pow((double)beta1, (double)step), bc2 = 1.0 - pow((double)beta2, (double)step);
  const float step_size = (float)((double)lr / bc1), inv_sqrt_bc2 = (float)(1.0 / sqrt(bc2));
  const float decay = 1.f - lr * weight_decay;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int per = dtype == ODY_BF16 ? 8 : 4;
  const int64_t nv = n / per;
  const unsigned blocks = (unsigned)std::min<int64_t>(std::max<int64_t>((nv + 255) / 256, 1), 256 * 16);
  ODY_BY_DTYPE(dtype,
               ODY_LAUNCH("adamw", st, adamw_kernel<bf16>, dim3(blocks), dim3(256), 0, (bf16*)param, (const bf16*)grad,
                          (bf16*)exp_avg, (bf16*)exp_avg_sq, n, decay, beta1, beta2, step_size, inv_sqrt_bc2, eps),
               ODY_LAUNCH("adamw", st, adamw_kernel<float>, dim3(blocks), dim3(256), 0, (float*)param, (const float*)grad,
                          (float*)exp_avg, (float*)exp_avg_sq, n, decay, beta1, beta2, step_size, inv_sqrt_bc2, eps));
  return ody_check_launch("adamw");
}
