// fp32 attention (forward and backward) on the vector ALUs, plus the delta
// pre-pass shared with the MFMA backward.
//
// These kernels serve the fp32 configuration, whose 1e-4 tolerance rules out
// bf16 matrix cores.  One thread owns one query row (forward, dQ) or one key row
// (dK, dV); the other side is staged through LDS as fp32 and read with
// wavefront-uniform (broadcast) 16-byte reads.  Everything is deterministic:
// no atomics, fixed summation order.
#include "attn_params.h"

namespace {

constexpr int SIMT_ROWS = 64;  // rows per block = one wavefront
constexpr int SIMT_TILE = 32;  // rows of the streamed side per LDS tile

template <typename T, int D>
__device__ __forceinline__ void stage_tile(float* dst, const T* src, int64_t stride_l, int row0, int nrows_valid,
                                           int tid) {
  // dst [SIMT_TILE][D] fp32; rows >= nrows_valid are zero-filled
  for (int e = tid; e < SIMT_TILE * D; e += SIMT_ROWS) {
    const int r = e / D, c = e % D;
    dst[e] = (r < nrows_valid) ? to_f32<T>(src[(int64_t)(row0 + r) * stride_l + c]) : 0.f;
  }
}

template <typename T, int D>
__global__ __launch_bounds__(SIMT_ROWS) void attn_fwd_simt_kernel(const AttnParams p) {
  __shared__ __attribute__((aligned(16))) float Ks[SIMT_TILE * D];
  __shared__ __attribute__((aligned(16))) float Vs[SIMT_TILE * D];
  const int tid = threadIdx.x;
  const int h = blockIdx.y, b = blockIdx.z, hk = h / p.group;
  const int q0 = blockIdx.x * SIMT_ROWS, qi = q0 + tid;
  const T* qp = static_cast<const T*>(p.q) + b * p.sq.b + h * p.sq.h;
  const T* kp = static_cast<const T*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const T* vp = static_cast<const T*>(p.v) + b * p.sv.b + hk * p.sv.h;

  float q[D], o[D];
#pragma unroll
  for (int d = 0; d < D; d++) {
    q[d] = (qi < p.Lq) ? to_f32<T>(qp[(int64_t)qi * p.sq.l + d]) : 0.f;
    o[d] = 0.f;
  }
  float m = -INFINITY, l = 0.f;
  const int lim = p.causal ? min(p.Lk - 1, qi + p.off) : p.Lk - 1;
  const int q_hi = min(q0 + SIMT_ROWS, p.Lq) - 1;
  int n_end = p.causal ? min(p.Lk, q_hi + p.off + 1) : p.Lk;
  if (n_end < 0) n_end = 0;

  for (int n0 = 0; n0 < n_end; n0 += SIMT_TILE) {
    const int valid = min(SIMT_TILE, p.Lk - n0);
    __syncthreads();
    stage_tile<T, D>(Ks, kp, p.sk.l, n0, valid, tid);
    stage_tile<T, D>(Vs, vp, p.sv.l, n0, valid, tid);
    __syncthreads();
    float s[SIMT_TILE];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < SIMT_TILE; j++) {
      float acc = 0.f;
#pragma unroll
      for (int d = 0; d < D; d += 4) {
        const f32x4 kv = *reinterpret_cast<const f32x4*>(Ks + j * D + d);
        acc = fmaf(q[d], kv[0], acc);
        acc = fmaf(q[d + 1], kv[1], acc);
        acc = fmaf(q[d + 2], kv[2], acc);
        acc = fmaf(q[d + 3], kv[3], acc);
      }
      acc *= p.scale;
      if (n0 + j > lim) acc = -INFINITY;
      s[j] = acc;
      mx = fmaxf(mx, acc);
    }
    const float m_new = fmaxf(m, mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __expf(m - m_use);
    m = m_new;
    l *= alpha;
#pragma unroll
    for (int d = 0; d < D; d++) o[d] *= alpha;
#pragma unroll
    for (int j = 0; j < SIMT_TILE; j++) {
      const float e = __expf(s[j] - m_use);
      l += e;
#pragma unroll
      for (int d = 0; d < D; d += 4) {
        const f32x4 vv = *reinterpret_cast<const f32x4*>(Vs + j * D + d);
        o[d] = fmaf(e, vv[0], o[d]);
        o[d + 1] = fmaf(e, vv[1], o[d + 1]);
        o[d + 2] = fmaf(e, vv[2], o[d + 2]);
        o[d + 3] = fmaf(e, vv[3], o[d + 3]);
      }
    }
  }
  if (qi < p.Lq) {
    T* op = static_cast<T*>(p.out) + b * p.so.b + h * p.so.h + (int64_t)qi * p.so.l;
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int d = 0; d < D; d++) op[d] = from_f32<T>(o[d] * inv);
    p.lse[((int64_t)b * p.Hq + h) * p.Lq + qi] = l > 0.f ? m + logf(l) : -INFINITY;
  }
}

// dQ: one thread per query row, keys streamed.
template <typename T, int D>
__global__ __launch_bounds__(SIMT_ROWS) void attn_bwd_dq_simt_kernel(const AttnParams p) {
  __shared__ __attribute__((aligned(16))) float Ks[SIMT_TILE * D];
  __shared__ __attribute__((aligned(16))) float Vs[SIMT_TILE * D];
  const int tid = threadIdx.x;
  const int h = blockIdx.y, b = blockIdx.z, hk = h / p.group;
  const int q0 = blockIdx.x * SIMT_ROWS, qi = q0 + tid;
  const T* qp = static_cast<const T*>(p.q) + b * p.sq.b + h * p.sq.h;
  const T* dop = static_cast<const T*>(p.dout) + b * p.sdo.b + h * p.sdo.h;
  const T* kp = static_cast<const T*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const T* vp = static_cast<const T*>(p.v) + b * p.sv.b + hk * p.sv.h;

  float q[D], dO[D], dq[D];
#pragma unroll
  for (int d = 0; d < D; d++) {
    q[d] = (qi < p.Lq) ? to_f32<T>(qp[(int64_t)qi * p.sq.l + d]) : 0.f;
    dO[d] = (qi < p.Lq) ? to_f32<T>(dop[(int64_t)qi * p.sdo.l + d]) : 0.f;
    dq[d] = 0.f;
  }
  const int64_t ri = ((int64_t)b * p.Hq + h) * p.Lq + qi;
  const float lse = (qi < p.Lq) ? p.lse[ri] : -INFINITY;
  const float delta = (qi < p.Lq) ? p.delta[ri] : 0.f;
  const int lim = (lse == -INFINITY) ? -1 : (p.causal ? min(p.Lk - 1, qi + p.off) : p.Lk - 1);
  const int q_hi = min(q0 + SIMT_ROWS, p.Lq) - 1;
  int n_end = p.causal ? min(p.Lk, q_hi + p.off + 1) : p.Lk;
  if (n_end < 0) n_end = 0;

  for (int n0 = 0; n0 < n_end; n0 += SIMT_TILE) {
    const int valid = min(SIMT_TILE, p.Lk - n0);
    __syncthreads();
    stage_tile<T, D>(Ks, kp, p.sk.l, n0, valid, tid);
    stage_tile<T, D>(Vs, vp, p.sv.l, n0, valid, tid);
    __syncthreads();
#pragma unroll 4
    for (int j = 0; j < SIMT_TILE; j++) {
      float s = 0.f, dp = 0.f;
#pragma unroll
      for (int d = 0; d < D; d += 4) {
        const f32x4 kv = *reinterpret_cast<const f32x4*>(Ks + j * D + d);
        const f32x4 vv = *reinterpret_cast<const f32x4*>(Vs + j * D + d);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          s = fmaf(q[d + e], kv[e], s);
          dp = fmaf(dO[d + e], vv[e], dp);
        }
      }
      const float pr = (n0 + j > lim) ? 0.f : __expf(s * p.scale - lse);
      const float ds = pr * (dp - delta) * p.scale;
#pragma unroll
      for (int d = 0; d < D; d += 4) {
        const f32x4 kv = *reinterpret_cast<const f32x4*>(Ks + j * D + d);
#pragma unroll
        for (int e = 0; e < 4; e++) dq[d + e] = fmaf(ds, kv[e], dq[d + e]);
      }
    }
  }
  if (qi < p.Lq) {
    T* dqp = static_cast<T*>(p.dq) + b * p.sdq.b + h * p.sdq.h + (int64_t)qi * p.sdq.l;
#pragma unroll
    for (int d = 0; d < D; d++) {
      float r = dq[d];
      if (p.accumulate_dq) r += to_f32<T>(dqp[d]);
      dqp[d] = from_f32<T>(r);
    }
  }
}

// dK (WHICH = 1) or dV (WHICH = 0): one thread per key row; the queries of every
// head of the group are streamed.
template <typename T, int D, int WHICH>
__global__ __launch_bounds__(SIMT_ROWS) void attn_bwd_dkv_simt_kernel(const AttnParams p) {
  __shared__ __attribute__((aligned(16))) float Qs[SIMT_TILE * D];
  __shared__ __attribute__((aligned(16))) float Os[SIMT_TILE * D];
  __shared__ float Ls[SIMT_TILE], Ds[SIMT_TILE];
  const int tid = threadIdx.x;
  const int hk = blockIdx.y, b = blockIdx.z;
  const int n0 = blockIdx.x * SIMT_ROWS, ki = n0 + tid;
  const T* kp = static_cast<const T*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const T* vp = static_cast<const T*>(p.v) + b * p.sv.b + hk * p.sv.h;

  float kreg[D], acc[D];
  float vreg[WHICH ? D : 1];
#pragma unroll
  for (int d = 0; d < D; d++) {
    kreg[d] = (ki < p.Lk) ? to_f32<T>(kp[(int64_t)ki * p.sk.l + d]) : 0.f;
    acc[d] = 0.f;
    if (WHICH) vreg[d] = (ki < p.Lk) ? to_f32<T>(vp[(int64_t)ki * p.sv.l + d]) : 0.f;
  }
  // first query that can see key n0 (the smallest key of this block)
  int i_begin = p.causal ? max(0, n0 - p.off) : 0;
  i_begin = (i_begin / SIMT_TILE) * SIMT_TILE;

  for (int hg = 0; hg < p.group; hg++) {
    const int h = hk * p.group + hg;
    const T* qp = static_cast<const T*>(p.q) + b * p.sq.b + h * p.sq.h;
    const T* dop = static_cast<const T*>(p.dout) + b * p.sdo.b + h * p.sdo.h;
    const int64_t rbase = ((int64_t)b * p.Hq + h) * p.Lq;
    for (int i0 = i_begin; i0 < p.Lq; i0 += SIMT_TILE) {
      const int valid = min(SIMT_TILE, p.Lq - i0);
      __syncthreads();
      stage_tile<T, D>(Qs, qp, p.sq.l, i0, valid, tid);
      stage_tile<T, D>(Os, dop, p.sdo.l, i0, valid, tid);
      if (tid < SIMT_TILE) {
        Ls[tid] = (tid < valid) ? p.lse[rbase + i0 + tid] : -INFINITY;
        Ds[tid] = (tid < valid) ? p.delta[rbase + i0 + tid] : 0.f;
      }
      __syncthreads();
#pragma unroll 4
      for (int j = 0; j < SIMT_TILE; j++) {
        const int qi = i0 + j;
        const float lse = Ls[j];
        float s = 0.f, dp = 0.f;
#pragma unroll
        for (int d = 0; d < D; d += 4) {
          const f32x4 qv = *reinterpret_cast<const f32x4*>(Qs + j * D + d);
#pragma unroll
          for (int e = 0; e < 4; e++) s = fmaf(qv[e], kreg[d + e], s);
          if (WHICH) {
            const f32x4 ov = *reinterpret_cast<const f32x4*>(Os + j * D + d);
#pragma unroll
            for (int e = 0; e < 4; e++) dp = fmaf(ov[e], vreg[d + e], dp);
          }
        }
        const bool masked = (lse == -INFINITY) || (p.causal && ki > qi + p.off);
        const float pr = masked ? 0.f : __expf(s * p.scale - lse);
        const float wgt = WHICH ? pr * (dp - Ds[j]) * p.scale : pr;
        const float* src = WHICH ? Qs : Os;
#pragma unroll
        for (int d = 0; d < D; d += 4) {
          const f32x4 xv = *reinterpret_cast<const f32x4*>(src + j * D + d);
#pragma unroll
          for (int e = 0; e < 4; e++) acc[d + e] = fmaf(wgt, xv[e], acc[d + e]);
        }
      }
    }
  }
  if (ki < p.Lk) {
    T* dst = WHICH ? static_cast<T*>(p.dk) + b * p.sdk.b + hk * p.sdk.h + (int64_t)ki * p.sdk.l
                   : static_cast<T*>(p.dv) + b * p.sdv.b + hk * p.sdv.h + (int64_t)ki * p.sdv.l;
#pragma unroll
    for (int d = 0; d < D; d++) dst[d] = from_f32<T>(acc[d]);
  }
}

// delta[b, h, i] = sum_d dO[b, i, h, d] * O[b, i, h, d]; LPR lanes per row,
// 16-byte loads.
template <typename T, int D>
__global__ __launch_bounds__(256) void attn_delta_kernel(const AttnParams p) {
  constexpr int VEC = Vec16B<T>::N, LPR = D / VEC, RPB = 256 / LPR;
  typedef typename Vec16B<T>::type vec_t;
  const int tid = threadIdx.x, sub = tid % LPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + tid / LPR;  // over B * Hq * Lq in (b, h, i) order
  const int64_t total = (int64_t)p.B * p.Hq * p.Lq;
  float acc = 0.f;
  if (row < total) {
    const int i = row % p.Lq;
    const int h = (row / p.Lq) % p.Hq;
    const int b = row / ((int64_t)p.Lq * p.Hq);
    const T* op = static_cast<const T*>(p.out) + b * p.so.b + h * p.so.h + (int64_t)i * p.so.l + sub * VEC;
    const T* dp = static_cast<const T*>(p.dout) + b * p.sdo.b + h * p.sdo.h + (int64_t)i * p.sdo.l + sub * VEC;
    const vec_t ov = *reinterpret_cast<const vec_t*>(op);
    const vec_t dv = *reinterpret_cast<const vec_t*>(dp);
#pragma unroll
    for (int e = 0; e < VEC; e++) acc = fmaf((float)ov[e], (float)dv[e], acc);
  }
#pragma unroll
  for (int s = LPR / 2; s > 0; s >>= 1) acc += __shfl_xor(acc, s, 64);
  if (row < total && sub == 0) p.delta[row] = acc;
}

template <typename T, int D>
int launch_fwd(const AttnParams& p, hipStream_t st) {
  dim3 grid((p.Lq + SIMT_ROWS - 1) / SIMT_ROWS, p.Hq, p.B);
  ODY_LAUNCH("attn_fwd_simt", st, (attn_fwd_simt_kernel<T, D>), grid, dim3(SIMT_ROWS), 0, p);
  return ody_check_launch("attn_fwd_simt");
}

template <typename T, int D>
int launch_bwd(const AttnParams& p, hipStream_t st) {
  dim3 gq((p.Lq + SIMT_ROWS - 1) / SIMT_ROWS, p.Hq, p.B);
  ODY_LAUNCH("attn_bwd_dq_simt", st, (attn_bwd_dq_simt_kernel<T, D>), gq, dim3(SIMT_ROWS), 0, p);
  int rc = ody_check_launch("attn_bwd_dq_simt");
  if (rc) return rc;
  dim3 gk((p.Lk + SIMT_ROWS - 1) / SIMT_ROWS, p.Hkv, p.B);
  ODY_LAUNCH("attn_bwd_dv_simt", st, (attn_bwd_dkv_simt_kernel<T, D, 0>), gk, dim3(SIMT_ROWS), 0, p);
  rc = ody_check_launch("attn_bwd_dv_simt");
  if (rc) return rc;
  ODY_LAUNCH("attn_bwd_dk_simt", st, (attn_bwd_dkv_simt_kernel<T, D, 1>), gk, dim3(SIMT_ROWS), 0, p);
  return ody_check_launch("attn_bwd_dk_simt");
}

template <typename T, int D>
int launch_delta(const AttnParams& p, hipStream_t st) {
  constexpr int RPB = 256 / (D / Vec16B<T>::N);
  const int64_t total = (int64_t)p.B * p.Hq * p.Lq;
  ODY_LAUNCH("attn_delta", st, (attn_delta_kernel<T, D>), dim3((unsigned)((total + RPB - 1) / RPB)), dim3(256), 0, p);
  return ody_check_launch("attn_delta");
}

}  // namespace

#define ODY_DISPATCH_T_D(FN)                                              \
  if (dtype == ODY_F32 && D == 64) return FN<float, 64>(p, st);           \
  if (dtype == ODY_F32 && D == 128) return FN<float, 128>(p, st);         \
  if (dtype == ODY_BF16 && D == 64) return FN<bf16, 64>(p, st);           \
  if (dtype == ODY_BF16 && D == 128) return FN<bf16, 128>(p, st);         \
  ody_set_error("attention: head_dim %d / dtype %d not built", D, dtype); \
  return ODY_ERR_UNSUPPORTED;

int ody_launch_attn_fwd_simt(const AttnParams& p, int D, int dtype, hipStream_t st) { ODY_DISPATCH_T_D(launch_fwd) }
int ody_launch_attn_bwd_simt(const AttnParams& p, int D, int dtype, hipStream_t st) { ODY_DISPATCH_T_D(launch_bwd) }
int ody_launch_attn_delta(const AttnParams& p, int D, int dtype, hipStream_t st) { ODY_DISPATCH_T_D(launch_delta) }
