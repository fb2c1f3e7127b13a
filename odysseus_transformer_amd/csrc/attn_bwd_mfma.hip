// Flash-attention backward for gfx950, bf16 in, fp32 accumulate, deterministic.
//
// Two kernels, no atomics:
//
//  * dK/dV kernel -- key-stationary.  A workgroup owns 128 keys of one kv head
//    (32 per wavefront, held in registers as B operands), loops over the query
//    heads of its group and streams query tiles (Q, dO, lse, delta) through LDS.
//      S  (q x k) = Q . K^T        dP (q x k) = dO . V^T
//      P = exp2(S*c - lse*log2e)   dS = P * (dP - delta)
//      dV^T (d x k) += dO^T . P    dK^T (d x k) += Q^T . dS
//    P and dS are accumulator tiles whose rows are the contraction index of the
//    next product, which is exactly the B-operand layout: they stay in registers.
//    Q^T / dO^T come from the same LDS tiles through the transpose read.
//
//  * dQ kernel -- query-stationary, the mirror image with every tile transposed.
//      S^T (k x q) = K . Q^T       dP^T = V . dO^T
//      dQ^T (d x q) += K^T . dS^T
//
// Recomputing S in both kernels costs 7 tile products instead of 5 but needs no
// fp32 dQ workspace, no atomics and no LDS round trip for P / dS.
//
// Row permutation: the 32 rows of an LDS-fed A operand are assigned to tile rows
// through kap() (swap of the two low 2-bit fields of the row index), so that the
// 4 rows touched by one transpose read are 4 tile rows apart.  With a row pitch
// of D + 8 elements both the 16-byte row reads and the transpose reads then spread
// over all LDS banks.
#include "attn_params.h"

namespace {

__device__ __forceinline__ int kap(int rho) { return (rho & ~15) | ((rho & 3) << 2) | ((rho >> 2) & 3); }
__device__ __forceinline__ int rho_of(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

// Copies a ROWS x D tile (row-major, row stride `stride`) into registers; rows at
// or beyond `limit` read as zero.
template <int ROWS, int D>
struct TileRegs {
  static constexpr int CPR = D / 8, N = ROWS * CPR / 256;
  bf16x8 r[N];
  __device__ __forceinline__ void load(const bf16* base, int64_t stride, int row0, int limit, int tid) {
#pragma unroll
    for (int j = 0; j < N; j++) {
      const int c = tid + 256 * j, row = c / CPR, col = (c % CPR) * 8;
      if (row0 + row < limit) r[j] = *reinterpret_cast<const bf16x8*>(base + (int64_t)(row0 + row) * stride + col);
      else r[j] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  __device__ __forceinline__ void store(bf16* lds, int tid) const {
#pragma unroll
    for (int j = 0; j < N; j++) {
      const int c = tid + 256 * j, row = c / CPR, col = (c % CPR) * 8;
      *reinterpret_cast<bf16x8*>(lds + row * (D + 8) + col) = r[j];
    }
  }
};

// A operand (rows = 32 consecutive-in-kap tile rows starting at row32, k = 16ks..16ks+15)
template <int D>
__device__ __forceinline__ bf16x8 lds_row_frag(const bf16* tile, int row32, int ks, int g, int i) {
  return *reinterpret_cast<const bf16x8*>(tile + (row32 + kap(i)) * (D + 8) + 16 * ks + 8 * g);
}

// A operand of the transposed tile: row = column (32*dt + i) of the LDS tile,
// k-index t <-> tile row kap(16*ss + 8*(t/4) + 4g + t%4) of the 32-row group.
template <int D>
__device__ __forceinline__ bf16x8 lds_tr_frag(const bf16* tile, int row32, int ss, int dt, int g, int i) {
  const int t = (i & 15) >> 2, col = 32 * dt + 16 * (i >> 4) + 4 * (i & 3);
  const bf16* p0 = tile + (row32 + 16 * ss + 4 * t + g) * (D + 8) + col;
  return concat4(lds_read_tr16(p0), lds_read_tr16(p0 + 2 * (D + 8)));
}

// ---------------------------------------------------------------------------
// dK / dV
// ---------------------------------------------------------------------------
// DROP (both kernels): attention dropout as the forward applied it (ody_dropout_hash): dV takes the kept entries of P
// scaled by 1 / (1 - p), and dP = dO V^T counts only where the entry was kept, with the same scale.
template <int D, bool DROP>
__global__ __launch_bounds__(256, 2) void attn_bwd_dkdv_kernel(const AttnParams p) {
  constexpr int BQ = 64, WK = 32, BN = 4 * WK, P = D + 8, KS = D / 16, DT = D / 32;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* Qs = reinterpret_cast<bf16*>(smem_raw);       // [2][BQ][P]
  bf16* Os = Qs + 2 * BQ * P;                         // [2][BQ][P]
  float* Ls = reinterpret_cast<float*>(Os + 2 * BQ * P);  // [2][BQ]  lse * log2e, in MFMA row order
  float* Ds = Ls + 2 * BQ;                            // [2][BQ]  delta, same order

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 5, i = lane & 31;
  const BlockCoord bc = ody_block_coord(p.Hkv, p.B);   // rank 0 = first key block = most query tiles
  const int hk = bc.h, b = bc.b;
  const int n0 = bc.rank * BN, wn0 = n0 + wave * WK, key = wn0 + i;
  const bf16* kp = static_cast<const bf16*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const bf16* vp = static_cast<const bf16*>(p.v) + b * p.sv.b + hk * p.sv.h;

  // this lane's key row of K and V as B operands (column = key, k = head dim)
  bf16x8 kf[KS], vf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    if (key < p.Lk) {
      kf[ks] = *reinterpret_cast<const bf16x8*>(kp + (int64_t)key * p.sk.l + 16 * ks + 8 * g);
      vf[ks] = *reinterpret_cast<const bf16x8*>(vp + (int64_t)key * p.sv.l + 16 * ks + 8 * g);
    } else {
      kf[ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      vf[ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  f32x16 dk[DT], dv[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) dk[dt][r] = dv[dt][r] = 0.f;

  int i_begin = p.causal ? max(0, n0 - p.off) : 0;
  i_begin = (i_begin / BQ) * BQ;
  const int ntq = (p.Lq > i_begin) ? (p.Lq - i_begin + BQ - 1) / BQ : 0;
  const int total = ntq * p.group;  // flattened (head-of-group, query tile) iteration space

  TileRegs<BQ, D> qr, dor;
  float lreg = 0.f, dreg = 0.f;
  auto gload = [&](int it) {
    const int hg = it / ntq, i0 = i_begin + (ntq - 1 - it % ntq) * BQ, h = hk * p.group + hg;
    const bf16* qp = static_cast<const bf16*>(p.q) + b * p.sq.b + h * p.sq.h;
    const bf16* dop = static_cast<const bf16*>(p.dout) + b * p.sdo.b + h * p.sdo.h;
    qr.load(qp, p.sq.l, i0, p.Lq, tid);
    dor.load(dop, p.sdo.l, i0, p.Lq, tid);
    if (tid < BQ) {
      const int qi = i0 + tid;
      const int64_t ri = ((int64_t)b * p.Hq + h) * p.Lq + qi;
      float l = (qi < p.Lq) ? p.lse[ri] : INFINITY;
      if (l == -INFINITY) l = INFINITY;  // a query that saw no key: P must be 0
      lreg = l * ODY_LOG2E;
      dreg = (qi < p.Lq) ? p.delta[ri] : 0.f;
    }
  };
  auto sstore = [&](int buf) {
    qr.store(Qs + buf * BQ * P, tid);
    dor.store(Os + buf * BQ * P, tid);
    if (tid < BQ) {
      const int pos = (tid & ~31) + kap(tid & 31);
      Ls[buf * BQ + pos] = lreg;
      Ds[buf * BQ + pos] = dreg;
    }
  };

  if (total > 0) {
    gload(0);
    sstore(0);
  }
  __syncthreads();
  const float c2 = p.scale_log2e;

  for (int it = 0; it < total; it++) {
    const int buf = it & 1;
    const unsigned dh = DROP ? ody_dropout_head(p.drop_seed, b * p.Hq + hk * p.group + it / ntq) : 0u;
    const int i0 = i_begin + (ntq - 1 - it % ntq) * BQ;   // last query tile first: the key blocks running on an XCD then read the same Q / dO tiles together
    if (it + 1 < total) gload(it + 1);
    const bf16* Qb = Qs + buf * BQ * P;
    const bf16* Ob = Os + buf * BQ * P;
#pragma unroll
    for (int mt = 0; mt < BQ / 32; mt++) {
      const int m0 = i0 + 32 * mt;
      // every query of this sub-tile is before every key of this wavefront: nothing to do
      const bool active = (m0 < p.Lq) && (!p.causal || (m0 + 31 + p.off >= wn0));
      if (!active) continue;
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        s = mfma32(lds_row_frag<D>(Qb, 32 * mt, ks, g, i), kf[ks], s);
        dp = mfma32(lds_row_frag<D>(Ob, 32 * mt, ks, g, i), vf[ks], dp);
      }
      const bool need_mask = p.causal && (m0 + p.off < wn0 + 31);
      bf16x8 pf[2], dsf[2];
#pragma unroll
      for (int a = 0; a < 4; a++) {
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(Ls + buf * BQ + 32 * mt + 8 * a + 4 * g);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(Ds + buf * BQ + 32 * mt + 8 * a + 4 * g);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int r = 4 * a + e;
          float pr = ody_exp2(fmaf(s[r], c2, -l4[e]));
          if (need_mask) {
            const int qi = m0 + kap(rho_of(r, g));
            if (key > qi + p.off) pr = 0.f;
          }
          float dpv = dp[r], pv = pr;
          if (DROP) {
            const bool keep = ody_dropout_hash(ody_dropout_row(dh, m0 + kap(rho_of(r, g))), key) >= p.drop_thresh;
            dpv = keep ? dpv * p.drop_scale : 0.f;
            pv = keep ? pr : 0.f;
          }
          const float dsv = pr * (dpv - d4[e]);
          pf[r >> 3][r & 7] = (bf16)pv;
          dsf[r >> 3][r & 7] = (bf16)dsv;
        }
      }
#pragma unroll
      for (int dt = 0; dt < DT; dt++) {
#pragma unroll
        for (int ss = 0; ss < 2; ss++) {
          dv[dt] = mfma32(lds_tr_frag<D>(Ob, 32 * mt, ss, dt, g, i), pf[ss], dv[dt]);
          dk[dt] = mfma32(lds_tr_frag<D>(Qb, 32 * mt, ss, dt, g, i), dsf[ss], dk[dt]);
        }
      }
    }
    if (it + 1 < total) sstore(buf ^ 1);
    __syncthreads();
  }

  if (key < p.Lk) {
    bf16* dkp = static_cast<bf16*>(p.dk) + b * p.sdk.b + hk * p.sdk.h + (int64_t)key * p.sdk.l;
    bf16* dvp = static_cast<bf16*>(p.dv) + b * p.sdv.b + hk * p.sdv.h + (int64_t)key * p.sdv.l;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int a = 0; a < 4; a++) {
        bf16x4 wk, wv;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          wk[e] = (bf16)(dk[dt][4 * a + e] * p.scale);
          wv[e] = (bf16)(DROP ? dv[dt][4 * a + e] * p.drop_scale : dv[dt][4 * a + e]);
        }
        *reinterpret_cast<bf16x4*>(dkp + 32 * dt + 8 * a + 4 * g) = wk;
        *reinterpret_cast<bf16x4*>(dvp + 32 * dt + 8 * a + 4 * g) = wv;
      }
  }
}

// ---------------------------------------------------------------------------
// dQ
// ---------------------------------------------------------------------------
template <int D, bool DROP>
__global__ __launch_bounds__(256) void attn_bwd_dq_kernel(const AttnParams p) {
  constexpr int BN = 64, WQ = 32, BM = 4 * WQ, P = D + 8, KS = D / 16, DT = D / 32;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* Ks = reinterpret_cast<bf16*>(smem_raw);  // [2][BN][P]
  bf16* Vs = Ks + 2 * BN * P;                    // [2][BN][P]

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 5, i = lane & 31;
  const BlockCoord bc = ody_block_coord(p.Hq, p.B);
  const int nqb = gridDim.x / (p.Hq * p.B);
  const int qblk = p.causal ? (nqb - 1 - bc.rank) : bc.rank;   // heaviest blocks first
  const int h = bc.h, b = bc.b, hk = h / p.group;
  const int q0 = qblk * BM, wq0 = q0 + wave * WQ, qi = wq0 + i;
  const bf16* qp = static_cast<const bf16*>(p.q) + b * p.sq.b + h * p.sq.h;
  const bf16* dop = static_cast<const bf16*>(p.dout) + b * p.sdo.b + h * p.sdo.h;
  const bf16* kp = static_cast<const bf16*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const bf16* vp = static_cast<const bf16*>(p.v) + b * p.sv.b + hk * p.sv.h;

  bf16x8 qf[KS], dof[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    if (qi < p.Lq) {
      qf[ks] = *reinterpret_cast<const bf16x8*>(qp + (int64_t)qi * p.sq.l + 16 * ks + 8 * g);
      dof[ks] = *reinterpret_cast<const bf16x8*>(dop + (int64_t)qi * p.sdo.l + 16 * ks + 8 * g);
    } else {
      qf[ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      dof[ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  const int64_t ri = ((int64_t)b * p.Hq + h) * p.Lq + qi;
  float lse2 = (qi < p.Lq) ? p.lse[ri] : INFINITY;
  if (lse2 == -INFINITY) lse2 = INFINITY;
  lse2 *= ODY_LOG2E;
  const float delta = (qi < p.Lq) ? p.delta[ri] : 0.f;
  const int lim = p.causal ? min(p.Lk - 1, qi + p.off) : p.Lk - 1;
  const unsigned drow = DROP ? ody_dropout_row(ody_dropout_head(p.drop_seed, b * p.Hq + h), qi) : 0u;

  f32x16 dq[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq[dt][r] = 0.f;

  const int q_hi = min(q0 + BM, p.Lq) - 1;
  int n_end = p.causal ? min(p.Lk, q_hi + p.off + 1) : p.Lk;
  if (n_end < 0) n_end = 0;
  const int ntiles = (n_end + BN - 1) / BN;

  TileRegs<BN, D> kr, vr;
  if (ntiles > 0) {
    kr.load(kp, p.sk.l, 0, p.Lk, tid);
    vr.load(vp, p.sv.l, 0, p.Lk, tid);
    kr.store(Ks, tid);
    vr.store(Vs, tid);
  }
  __syncthreads();
  const float c2 = p.scale_log2e;

  for (int t = 0; t < ntiles; t++) {
    const int buf = t & 1, n0 = t * BN;
    if (t + 1 < ntiles) {
      kr.load(kp, p.sk.l, n0 + BN, p.Lk, tid);
      vr.load(vp, p.sv.l, n0 + BN, p.Lk, tid);
    }
    const bf16* Kb = Ks + buf * BN * P;
    const bf16* Vb = Vs + buf * BN * P;
#pragma unroll
    for (int kt = 0; kt < BN / 32; kt++) {
      const int k0 = n0 + 32 * kt;
      const bool active = (k0 < p.Lk) && (!p.causal || (k0 <= wq0 + WQ - 1 + p.off));
      if (!active) continue;
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        s = mfma32(lds_row_frag<D>(Kb, 32 * kt, ks, g, i), qf[ks], s);
        dp = mfma32(lds_row_frag<D>(Vb, 32 * kt, ks, g, i), dof[ks], dp);
      }
      const bool need_mask = (k0 + 32 > p.Lk) || (p.causal && (k0 + 31 > wq0 + p.off));
      bf16x8 dsf[2];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        float pr = ody_exp2(fmaf(s[r], c2, -lse2));
        if (need_mask) {
          const int kj = k0 + kap(rho_of(r, g));
          if (kj > lim) pr = 0.f;
        }
        float dpv = dp[r];
        if (DROP) dpv = ody_dropout_hash(drow, k0 + kap(rho_of(r, g))) >= p.drop_thresh ? dpv * p.drop_scale : 0.f;
        dsf[r >> 3][r & 7] = (bf16)(pr * (dpv - delta));
      }
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int ss = 0; ss < 2; ss++) dq[dt] = mfma32(lds_tr_frag<D>(Kb, 32 * kt, ss, dt, g, i), dsf[ss], dq[dt]);
    }
    if (t + 1 < ntiles) {
      kr.store(Ks + (buf ^ 1) * BN * P, tid);
      vr.store(Vs + (buf ^ 1) * BN * P, tid);
    }
    __syncthreads();
  }

  if (qi < p.Lq && p.dq_f32) {
    float* dqp = static_cast<float*>(p.dq) + b * p.sdq.b + h * p.sdq.h + (int64_t)qi * p.sdq.l;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int a = 0; a < 4; a++) {
        f32x4* dst = reinterpret_cast<f32x4*>(dqp + 32 * dt + 8 * a + 4 * g);
        f32x4 w = {0.f, 0.f, 0.f, 0.f};
        if (p.accumulate_dq) w = *dst;
#pragma unroll
        for (int e = 0; e < 4; e++) w[e] += dq[dt][4 * a + e] * p.scale;
        *dst = w;
      }
  } else if (qi < p.Lq) {
    bf16* dqp = static_cast<bf16*>(p.dq) + b * p.sdq.b + h * p.sdq.h + (int64_t)qi * p.sdq.l;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int a = 0; a < 4; a++) {
        bf16x4* dst = reinterpret_cast<bf16x4*>(dqp + 32 * dt + 8 * a + 4 * g);
        bf16x4 w;
        bf16x4 old = {0, 0, 0, 0};
        if (p.accumulate_dq) old = *dst;
#pragma unroll
        for (int e = 0; e < 4; e++) w[e] = (bf16)(dq[dt][4 * a + e] * p.scale + (float)old[e]);
        *dst = w;
      }
  }
}

template <int D, bool DROP>
int launch(const AttnParams& p, hipStream_t st) {
  constexpr size_t smem_kv = (size_t)2 * 2 * 64 * (D + 8) * sizeof(bf16) + 2 * 2 * 64 * sizeof(float);
  constexpr size_t smem_q = (size_t)2 * 2 * 64 * (D + 8) * sizeof(bf16);
  if (int rc = ody_allow_dynamic_lds(reinterpret_cast<const void*>(&attn_bwd_dkdv_kernel<D, DROP>), smem_kv, "attn_bwd"))
    return rc;
  if (int rc = ody_allow_dynamic_lds(reinterpret_cast<const void*>(&attn_bwd_dq_kernel<D, DROP>), smem_q, "attn_bwd"))
    return rc;
  dim3 gk(((p.Lk + 127) / 128) * p.Hkv * p.B);
  ODY_LAUNCH("attn_bwd_dkdv", st, (attn_bwd_dkdv_kernel<D, DROP>), gk, dim3(256), smem_kv, p);
  int rc = ody_check_launch("attn_bwd_dkdv");
  if (rc) return rc;
  dim3 gq(((p.Lq + 127) / 128) * p.Hq * p.B);
  ODY_LAUNCH("attn_bwd_dq", st, (attn_bwd_dq_kernel<D, DROP>), gq, dim3(256), smem_q, p);
  return ody_check_launch("attn_bwd_dq");
}

}  // namespace

int ody_launch_attn_bwd_mfma(const AttnParams& p, int D, hipStream_t st) {
  if (p.drop_thresh != 0) {   // dropout: these kernels serve both head dims
    if (D == 64) return launch<64, true>(p, st);
    if (D == 128) return launch<128, true>(p, st);
  } else if (D == 64) {
    return launch<64, false>(p, st);   // head_dim 128 has its own kernels (attn_bwd_pipe.hip)
  }
  ody_set_error("attn_bwd: head_dim %d not built here", D);
  return ODY_ERR_UNSUPPORTED;
}
