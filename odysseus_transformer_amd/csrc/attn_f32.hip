// fp32 attention (forward and backward) on the fp32 matrix cores, plus the delta
// pre-pass shared with the bf16 backward.
//
// These kernels serve the fp32 configuration, whose 1e-4 tolerance rules out bf16
// operands.  All products run on v_mfma_f32_32x32x2_f32 (lane = 32 g + i holds
// A[row i][k = g] and B[k = g][col i]; the 32 x 32 result sits in 16 registers,
// register r of lane (i, g) = row 8 (r / 4) + 4 g + r % 4, column i).
//
// A workgroup is 4 wavefronts of 32 rows each (queries in the forward and dQ kernels,
// keys in the dK / dV kernel); the other side is streamed in tiles of 32 rows through
// LDS, the next tile being fetched into registers while the current one is multiplied.
// As in the bf16 kernels the score tile is computed transposed where the wavefront owns
// queries (S^T = K Q^T), so one lane = one query and softmax statistics need no
// cross-lane traffic beyond one swap of the wavefront halves, and the result registers
// are directly the B operand of the next product.
//
// Two index permutations keep every LDS read conflict-free and 16 bytes wide where it
// can be:
//  * contraction over head_dim: k-step 4 j + t multiplies element 8 j + 4 g + t, so the
//    streamed operand is one 16-byte read per four MFMAs and the resident operand is
//    loaded once in the same order;
//  * contraction over the 32 streamed rows: k-step ks multiplies row 8 (ks / 4) + 4 g +
//    ks % 4, which is the row that result register ks of this lane already holds.
// Everything is deterministic: no atomics, fixed summation order.
#include "attn_params.h"
#include "attn_tile.h"

namespace {

constexpr int F_WAVES = 4;
constexpr int F_THREADS = 64 * F_WAVES;
constexpr int F_ROWS = 32 * F_WAVES;  // rows owned by a workgroup
constexpr int F_TILE = 32;            // rows of the streamed side per LDS tile
constexpr float LN2 = 0.6931471805599453f;

__device__ __forceinline__ f32x16 mfma_f32(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// row of a 32-row tile that result register r of a lane in half g holds
__device__ __forceinline__ int acc_row(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

// One 32-row tile of a (rows, D) fp32 matrix on its way from global memory to LDS:
// D / 32 16-byte pieces per thread, rows past `nvalid` read as zero.
template <int D>
struct TileRegs {
  static constexpr int N = D / 32, LD = D + 4;
  f32x4 v[N];
  __device__ __forceinline__ void fetch(const float* src, int64_t stride, int row0, int nvalid, int tid) {
#pragma unroll
    for (int c = 0; c < N; c++) {
      const int e = tid + c * F_THREADS, r = e / (D / 4), x = e % (D / 4);
      v[c] = (r < nvalid) ? *reinterpret_cast<const f32x4*>(src + (int64_t)(row0 + r) * stride + 4 * x)
                          : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }
  __device__ __forceinline__ void put(float* dst, int tid) const {
#pragma unroll
    for (int c = 0; c < N; c++) {
      const int e = tid + c * F_THREADS, r = e / (D / 4), x = e % (D / 4);
      *reinterpret_cast<f32x4*>(dst + r * LD + 4 * x) = v[c];
    }
  }
};

// The resident operand of a head_dim contraction: row `row` of a (rows, D) matrix in
// k-step order (element 4 j + t = column 8 j + 4 g + t), times `mul`.
template <int D>
__device__ __forceinline__ void load_row_frag(float (&f)[D / 2], const float* base, int64_t stride, int row, bool ok,
                                              int g, float mul) {
#pragma unroll
  for (int j = 0; j < D / 8; j++) {
    const f32x4 v = ok ? *reinterpret_cast<const f32x4*>(base + (int64_t)row * stride + 8 * j + 4 * g)
                       : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < 4; t++) f[4 * j + t] = v[t] * mul;
  }
}

// acc (+)= T F^T for a 32-row LDS tile T (rows = MFMA rows) and a resident fragment F;
// two accumulation chains, summed by the caller.
template <int D>
__device__ __forceinline__ void tile_times_frag(const float* tile, int i, int g, const float (&f)[D / 2], f32x16& c0,
                                                f32x16& c1) {
  constexpr int LD = D + 4;
#pragma unroll
  for (int j = 0; j < D / 8; j++) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(tile + i * LD + 8 * j + 4 * g);
#pragma unroll
    for (int t = 0; t < 4; t++) {
      if (j & 1) c1 = mfma_f32(a[t], f[4 * j + t], c1);
      else c0 = mfma_f32(a[t], f[4 * j + t], c0);
    }
  }
}

// Two products of that kind at once, interleaved: each is the other's independent chain.
template <int D>
__device__ __forceinline__ void tiles_times_frags(const float* ta, const float (&fa)[D / 2], f32x16& ca, const float* tb,
                                                  const float (&fb)[D / 2], f32x16& cb, int i, int g) {
  constexpr int LD = D + 4;
#pragma unroll
  for (int j = 0; j < D / 8; j++) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(ta + i * LD + 8 * j + 4 * g);
    const f32x4 b = *reinterpret_cast<const f32x4*>(tb + i * LD + 8 * j + 4 * g);
#pragma unroll
    for (int t = 0; t < 4; t++) {
      ca = mfma_f32(a[t], fa[4 * j + t], ca);
      cb = mfma_f32(b[t], fb[4 * j + t], cb);
    }
  }
}

// acc[db] += T^T W for a 32-row LDS tile T (its 32 rows are contracted) and the weights
// W held in result-register order; D / 32 independent chains.
template <int D>
__device__ __forceinline__ void tile_t_times_regs(const float* tile, int i, int g, const f32x16& w,
                                                  f32x16 (&acc)[D / 32]) {
  constexpr int LD = D + 4;
#pragma unroll
  for (int ks = 0; ks < 16; ks++) {
    const float* row = tile + acc_row(ks, g) * LD + i;
#pragma unroll
    for (int db = 0; db < D / 32; db++) acc[db] = mfma_f32(row[32 * db], w[ks], acc[db]);
  }
}

// acc[db][r] is element (row i of the owner, column 32 db + 8 (r / 4) + 4 g + r % 4):
// four consecutive columns per register quad -> one 16-byte store each.
template <int D>
__device__ __forceinline__ void store_rows(float* dst, const f32x16 (&acc)[D / 32], int g, float mul, bool add) {
#pragma unroll
  for (int db = 0; db < D / 32; db++)
#pragma unroll
    for (int a = 0; a < 4; a++) {
      f32x4* out = reinterpret_cast<f32x4*>(dst + 32 * db + 8 * a + 4 * g);
      f32x4 v{acc[db][4 * a] * mul, acc[db][4 * a + 1] * mul, acc[db][4 * a + 2] * mul, acc[db][4 * a + 3] * mul};
      if (add) v += *out;
      *out = v;
    }
}

// ---------------------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------------------
// DROP (all three kernels): attention dropout (AttnParams::drop_*, ody_dropout_hash): row sums and lse are those of the
// full P; the entries that enter P V are the kept ones scaled by 1 / (1 - p), and dP counts only where an entry was kept.
template <int D, bool DROP>
__global__ __launch_bounds__(F_THREADS, D == 64 ? 3 : 1) void attn_fwd_f32_kernel(const AttnParams p) {
  constexpr int LD = D + 4, NDB = D / 32;
  __shared__ __attribute__((aligned(16))) float Ks[F_TILE * LD];
  __shared__ __attribute__((aligned(16))) float Vs[F_TILE * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i = lane & 31, g = lane >> 5;
  const BlockCoord bc = ody_block_coord(p.Hq, p.B);
  const int nqb = gridDim.x / (p.Hq * p.B);
  const int qblk = p.causal ? (nqb - 1 - bc.rank) : bc.rank;  // heaviest blocks first
  const int h = bc.h, b = bc.b, hk = h / p.group;
  const int q0 = qblk * F_ROWS, wq0 = q0 + wave * 32, qi = wq0 + i;
  const float* qp = static_cast<const float*>(p.q) + b * p.sq.b + h * p.sq.h;
  const float* kp = static_cast<const float*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const float* vp = static_cast<const float*>(p.v) + b * p.sv.b + hk * p.sv.h;

  float qf[D / 2];  // scores come out in the log2 domain
  load_row_frag<D>(qf, qp, p.sq.l, qi, qi < p.Lq, g, p.scale_log2e);
  f32x16 o[NDB];
#pragma unroll
  for (int db = 0; db < NDB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[db][r] = 0.f;
  float m = -INFINITY, l = 0.f;
  const unsigned drow = DROP ? ody_dropout_row(ody_dropout_head(p.drop_seed, b * p.Hq + h), qi) : 0u;

  // last key this lane's query sees, the first query of the wavefront sees, and the
  // key ranges the workgroup and the wavefront have to walk
  const int lim = p.causal ? min(p.Lk - 1, qi + p.off) : p.Lk - 1;
  const int lim_first = p.causal ? min(p.Lk - 1, wq0 + p.off) : p.Lk - 1;
  const int blk_hi = min(q0 + F_ROWS, p.Lq) - 1, wav_hi = min(wq0 + 32, p.Lq) - 1;
  const int n_end = max(0, p.causal ? min(p.Lk, blk_hi + p.off + 1) : p.Lk);
  const int w_end = (wq0 < p.Lq) ? max(0, p.causal ? min(p.Lk, wav_hi + p.off + 1) : p.Lk) : 0;

  TileRegs<D> kr, vr;
  if (n_end > 0) {
    kr.fetch(kp, p.sk.l, 0, min(F_TILE, p.Lk), tid);
    vr.fetch(vp, p.sv.l, 0, min(F_TILE, p.Lk), tid);
  }
  for (int n0 = 0; n0 < n_end; n0 += F_TILE) {
    __syncthreads();
    kr.put(Ks, tid);
    vr.put(Vs, tid);
    __syncthreads();
    if (n0 + F_TILE < n_end) {
      kr.fetch(kp, p.sk.l, n0 + F_TILE, min(F_TILE, p.Lk - n0 - F_TILE), tid);
      vr.fetch(vp, p.sv.l, n0 + F_TILE, min(F_TILE, p.Lk - n0 - F_TILE), tid);
    }
    if (n0 >= w_end) continue;  // wavefront-uniform: nothing visible to this wavefront here

    f32x16 s, s1;
#pragma unroll
    for (int r = 0; r < 16; r++) s[r] = s1[r] = 0.f;
    tile_times_frag<D>(Ks, i, g, qf, s, s1);
    s += s1;
    if (n0 + F_TILE - 1 > lim_first) {
#pragma unroll
      for (int r = 0; r < 16; r++)
        if (n0 + acc_row(r, g) > lim) s[r] = -INFINITY;
    }
    float mx = s[0];
#pragma unroll
    for (int r = 1; r < 16; r++) mx = fmaxf(mx, s[r]);
    mx = half_swap_max(mx);
    const float m_new = fmaxf(m, mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = ody_exp2(m - m_use);
    m = m_new;
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      s[r] = ody_exp2(s[r] - m_use);
      sum += s[r];
      if (DROP && ody_dropout_hash(drow, n0 + acc_row(r, g)) < p.drop_thresh) s[r] = 0.f;
    }
    l = l * alpha + sum;
#pragma unroll
    for (int db = 0; db < NDB; db++) o[db] *= alpha;
    tile_t_times_regs<D>(Vs, i, g, s, o);
  }

  l = half_swap_sum(l);
  if (qi < p.Lq) {
    float* op = static_cast<float*>(p.out) + b * p.so.b + h * p.so.h + (int64_t)qi * p.so.l;
    store_rows<D>(op, o, g, l > 0.f ? (DROP ? p.drop_scale : 1.f) / l : 0.f, false);
    if (g == 0) p.lse[((int64_t)b * p.Hq + h) * p.Lq + qi] = l > 0.f ? (m + __log2f(l)) * LN2 : -INFINITY;
  }
}

// ---------------------------------------------------------------------------------------
// dQ: the wavefront owns 32 queries, keys are streamed
// ---------------------------------------------------------------------------------------
template <int D, bool DROP>
__global__ __launch_bounds__(F_THREADS) void attn_bwd_dq_f32_kernel(const AttnParams p) {
  constexpr int LD = D + 4, NDB = D / 32;
  __shared__ __attribute__((aligned(16))) float Ks[F_TILE * LD];
  __shared__ __attribute__((aligned(16))) float Vs[F_TILE * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i = lane & 31, g = lane >> 5;
  const BlockCoord bc = ody_block_coord(p.Hq, p.B);
  const int nqb = gridDim.x / (p.Hq * p.B);
  const int qblk = p.causal ? (nqb - 1 - bc.rank) : bc.rank;
  const int h = bc.h, b = bc.b, hk = h / p.group;
  const int q0 = qblk * F_ROWS, wq0 = q0 + wave * 32, qi = wq0 + i;
  const float* qp = static_cast<const float*>(p.q) + b * p.sq.b + h * p.sq.h;
  const float* dop = static_cast<const float*>(p.dout) + b * p.sdo.b + h * p.sdo.h;
  const float* kp = static_cast<const float*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const float* vp = static_cast<const float*>(p.v) + b * p.sv.b + hk * p.sv.h;

  float qf[D / 2], dof[D / 2];
  load_row_frag<D>(qf, qp, p.sq.l, qi, qi < p.Lq, g, p.scale_log2e);
  load_row_frag<D>(dof, dop, p.sdo.l, qi, qi < p.Lq, g, 1.f);
  const int64_t ri = ((int64_t)b * p.Hq + h) * p.Lq + qi;
  const float lse = (qi < p.Lq) ? p.lse[ri] : -INFINITY;
  const float lse2 = lse * ODY_LOG2E;
  const float delta = (qi < p.Lq) ? p.delta[ri] : 0.f;
  const unsigned drow = DROP ? ody_dropout_row(ody_dropout_head(p.drop_seed, b * p.Hq + h), qi) : 0u;
  // a query with no visible key (lse = -inf) contributes nothing
  const int lim = (lse == -INFINITY) ? -1 : (p.causal ? min(p.Lk - 1, qi + p.off) : p.Lk - 1);
  f32x16 dq[NDB];
#pragma unroll
  for (int db = 0; db < NDB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq[db][r] = 0.f;

  const int blk_hi = min(q0 + F_ROWS, p.Lq) - 1, wav_hi = min(wq0 + 32, p.Lq) - 1;
  const int n_end = max(0, p.causal ? min(p.Lk, blk_hi + p.off + 1) : p.Lk);
  const int w_end = (wq0 < p.Lq) ? max(0, p.causal ? min(p.Lk, wav_hi + p.off + 1) : p.Lk) : 0;

  TileRegs<D> kr, vr;
  if (n_end > 0) {
    kr.fetch(kp, p.sk.l, 0, min(F_TILE, p.Lk), tid);
    vr.fetch(vp, p.sv.l, 0, min(F_TILE, p.Lk), tid);
  }
  for (int n0 = 0; n0 < n_end; n0 += F_TILE) {
    __syncthreads();
    kr.put(Ks, tid);
    vr.put(Vs, tid);
    __syncthreads();
    if (n0 + F_TILE < n_end) {
      kr.fetch(kp, p.sk.l, n0 + F_TILE, min(F_TILE, p.Lk - n0 - F_TILE), tid);
      vr.fetch(vp, p.sv.l, n0 + F_TILE, min(F_TILE, p.Lk - n0 - F_TILE), tid);
    }
    if (n0 >= w_end) continue;

    f32x16 s, dp;
#pragma unroll
    for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
    tiles_times_frags<D>(Ks, qf, s, Vs, dof, dp, i, g);  // S^T = K Q^T (log2 domain), dP^T = V dO^T
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const float pr = (n0 + acc_row(r, g) > lim) ? 0.f : ody_exp2(s[r] - lse2);
      float dpv = dp[r];
      if (DROP) dpv = ody_dropout_hash(drow, n0 + acc_row(r, g)) >= p.drop_thresh ? dpv * p.drop_scale : 0.f;
      s[r] = pr * (dpv - delta) * p.scale;  // dS^T
    }
    tile_t_times_regs<D>(Ks, i, g, s, dq);  // dQ^T += K^T dS^T
  }
  if (qi < p.Lq) {
    float* dqp = static_cast<float*>(p.dq) + b * p.sdq.b + h * p.sdq.h + (int64_t)qi * p.sdq.l;
    store_rows<D>(dqp, dq, g, 1.f, p.accumulate_dq != 0);
  }
}

// ---------------------------------------------------------------------------------------
// dK / dV: the wavefront owns 32 keys, the queries of every head of the group are streamed.
// WHICH: 0 = dV only, 1 = dK only, 2 = both.  (At head_dim 128 the K and V fragments and both
// accumulators do not fit the register file together, so dV and dK take a pass each.)
// ---------------------------------------------------------------------------------------
template <int D, int WHICH, bool DROP>
__global__ __launch_bounds__(F_THREADS, (D == 64 || WHICH == 0) ? 2 : 1) void attn_bwd_dkdv_f32_kernel(const AttnParams p) {
  constexpr int LD = D + 4, NDB = D / 32;
  constexpr bool DO_DV = (WHICH != 1), DO_DK = (WHICH != 0);
  __shared__ __attribute__((aligned(16))) float Qs[F_TILE * LD];
  __shared__ __attribute__((aligned(16))) float Os[F_TILE * LD];
  __shared__ __attribute__((aligned(16))) float Ls[F_TILE];  // lse in the log2 domain; +inf = row contributes nothing
  __shared__ __attribute__((aligned(16))) float Ds[F_TILE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i = lane & 31, g = lane >> 5;
  const BlockCoord bc = ody_block_coord(p.Hkv, p.B);
  const int kblk = bc.rank;  // with causal masking the first key block is the heaviest
  const int hk = bc.h, b = bc.b;
  const int n0 = kblk * F_ROWS, wn0 = n0 + wave * 32, ki = wn0 + i;
  const float* kp = static_cast<const float*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const float* vp = static_cast<const float*>(p.v) + b * p.sv.b + hk * p.sv.h;

  float kf[D / 2];
  float vf[DO_DK ? D / 2 : 1];
  load_row_frag<D>(kf, kp, p.sk.l, ki, ki < p.Lk, g, p.scale_log2e);
  if constexpr (DO_DK) load_row_frag<D>(vf, vp, p.sv.l, ki, ki < p.Lk, g, 1.f);
  f32x16 dk[DO_DK ? NDB : 1], dv[DO_DV ? NDB : 1];
#pragma unroll
  for (int db = 0; db < NDB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      if constexpr (DO_DK) dk[db][r] = 0.f;
      if constexpr (DO_DV) dv[db][r] = 0.f;
    }

  // first query tile that sees the first key of the workgroup / of the wavefront
  const int i_begin = p.causal ? (max(0, n0 - p.off) / F_TILE) * F_TILE : 0;
  const int w_begin = p.causal ? max(0, wn0 - p.off) : 0;

  TileRegs<D> qr, dor;
  float lr = 0.f, dr = 0.f;  // threads 0..31 carry lse and delta of the next tile
  for (int hg = 0; hg < p.group; hg++) {
    const int h = hk * p.group + hg;
    const float* qp = static_cast<const float*>(p.q) + b * p.sq.b + h * p.sq.h;
    const float* dop = static_cast<const float*>(p.dout) + b * p.sdo.b + h * p.sdo.h;
    const int64_t rbase = ((int64_t)b * p.Hq + h) * p.Lq;
    const unsigned dh = DROP ? ody_dropout_head(p.drop_seed, b * p.Hq + h) : 0u;
    auto fetch = [&](int i0) {
      const int valid = min(F_TILE, p.Lq - i0);
      qr.fetch(qp, p.sq.l, i0, valid, tid);
      dor.fetch(dop, p.sdo.l, i0, valid, tid);
      if (tid < F_TILE) {
        const float x = (tid < valid) ? p.lse[rbase + i0 + tid] : -INFINITY;
        lr = (x == -INFINITY) ? INFINITY : x * ODY_LOG2E;
        dr = (tid < valid) ? p.delta[rbase + i0 + tid] : 0.f;
      }
    };
    if (i_begin < p.Lq) fetch(i_begin);
    for (int i0 = i_begin; i0 < p.Lq; i0 += F_TILE) {
      __syncthreads();
      qr.put(Qs, tid);
      dor.put(Os, tid);
      if (tid < F_TILE) {
        Ls[tid] = lr;
        Ds[tid] = dr;
      }
      __syncthreads();
      if (i0 + F_TILE < p.Lq) fetch(i0 + F_TILE);
      if (i0 + F_TILE <= w_begin || wn0 >= p.Lk) continue;  // wavefront-uniform

      // S = Q K^T (log2 domain): rows = queries, column = this lane's key; dP = dO V^T
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
      if constexpr (DO_DK) {
        tiles_times_frags<D>(Qs, kf, s, Os, vf, dp, i, g);
      } else {
        tile_times_frag<D>(Qs, i, g, kf, s, dp);
        s += dp;
      }
      f32x4 lv[4], dl[4];
#pragma unroll
      for (int a = 0; a < 4; a++) {
        lv[a] = *reinterpret_cast<const f32x4*>(Ls + 8 * a + 4 * g);
        dl[a] = *reinterpret_cast<const f32x4*>(Ds + 8 * a + 4 * g);
      }
      const int vis = p.causal ? ki - p.off - i0 : -1;  // tile row r is masked iff r < vis
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float pr = (acc_row(r, g) < vis) ? 0.f : ody_exp2(s[r] - lv[r >> 2][r & 3]);
        bool keep = true;
        if (DROP) keep = ody_dropout_hash(ody_dropout_row(dh, i0 + acc_row(r, g)), ki) >= p.drop_thresh;
        s[r] = DROP ? (keep ? pr * p.drop_scale : 0.f) : pr;
        if constexpr (DO_DK) {
          const float dpv = DROP ? (keep ? dp[r] * p.drop_scale : 0.f) : dp[r];
          dp[r] = pr * (dpv - dl[r >> 2][r & 3]) * p.scale;  // dS
        }
      }
      if constexpr (DO_DV) tile_t_times_regs<D>(Os, i, g, s, dv);   // dV^T += dO^T P
      if constexpr (DO_DK) tile_t_times_regs<D>(Qs, i, g, dp, dk);  // dK^T += Q^T dS
    }
  }
  if (ki < p.Lk) {
    if constexpr (DO_DK) {
      float* dst = static_cast<float*>(p.dk) + b * p.sdk.b + hk * p.sdk.h + (int64_t)ki * p.sdk.l;
      store_rows<D>(dst, dk, g, 1.f, false);
    }
    if constexpr (DO_DV) {
      float* dst = static_cast<float*>(p.dv) + b * p.sdv.b + hk * p.sdv.h + (int64_t)ki * p.sdv.l;
      store_rows<D>(dst, dv, g, 1.f, false);
    }
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

template <int D, bool DROP>
int launch_fwd(const AttnParams& p, hipStream_t st) {
  const int nqb = (p.Lq + F_ROWS - 1) / F_ROWS;
  ODY_LAUNCH("attn_fwd_f32", st, (attn_fwd_f32_kernel<D, DROP>), dim3(nqb * p.Hq * p.B), dim3(F_THREADS), 0, p);
  return ody_check_launch("attn_fwd_f32");
}

template <int D, bool DROP>
int launch_bwd(const AttnParams& p, hipStream_t st) {
  const int nqb = (p.Lq + F_ROWS - 1) / F_ROWS, nkb = (p.Lk + F_ROWS - 1) / F_ROWS;
  const dim3 gk(nkb * p.Hkv * p.B), blk(F_THREADS);
  int rc;
  if constexpr (D == 64) {
    ODY_LAUNCH("attn_bwd_dkdv_f32", st, (attn_bwd_dkdv_f32_kernel<D, 2, DROP>), gk, blk, 0, p);
    if ((rc = ody_check_launch("attn_bwd_dkdv_f32"))) return rc;
  } else {
    ODY_LAUNCH("attn_bwd_dv_f32", st, (attn_bwd_dkdv_f32_kernel<D, 0, DROP>), gk, blk, 0, p);
    if ((rc = ody_check_launch("attn_bwd_dv_f32"))) return rc;
    ODY_LAUNCH("attn_bwd_dk_f32", st, (attn_bwd_dkdv_f32_kernel<D, 1, DROP>), gk, blk, 0, p);
    if ((rc = ody_check_launch("attn_bwd_dk_f32"))) return rc;
  }
  ODY_LAUNCH("attn_bwd_dq_f32", st, (attn_bwd_dq_f32_kernel<D, DROP>), dim3(nqb * p.Hq * p.B), blk, 0, p);
  return ody_check_launch("attn_bwd_dq_f32");
}

template <typename T, int D>
int launch_delta(const AttnParams& p, hipStream_t st) {
  constexpr int RPB = 256 / (D / Vec16B<T>::N);
  const int64_t total = (int64_t)p.B * p.Hq * p.Lq;
  ODY_LAUNCH("attn_delta", st, (attn_delta_kernel<T, D>), dim3((unsigned)((total + RPB - 1) / RPB)), dim3(256), 0, p);
  return ody_check_launch("attn_delta");
}

}  // namespace

int ody_launch_attn_fwd_f32(const AttnParams& p, int D, hipStream_t st) {
  const bool drop = p.drop_thresh != 0;
  if (D == 64) return drop ? launch_fwd<64, true>(p, st) : launch_fwd<64, false>(p, st);
  if (D == 128) return drop ? launch_fwd<128, true>(p, st) : launch_fwd<128, false>(p, st);
  ody_set_error("fp32 attention: head_dim %d not built", D);
  return ODY_ERR_UNSUPPORTED;
}

int ody_launch_attn_bwd_f32(const AttnParams& p, int D, hipStream_t st) {
  const bool drop = p.drop_thresh != 0;
  if (D == 64) return drop ? launch_bwd<64, true>(p, st) : launch_bwd<64, false>(p, st);
  if (D == 128) return drop ? launch_bwd<128, true>(p, st) : launch_bwd<128, false>(p, st);
  ody_set_error("fp32 attention: head_dim %d not built", D);
  return ODY_ERR_UNSUPPORTED;
}

int ody_launch_attn_delta(const AttnParams& p, int D, int dtype, hipStream_t st) {
  if (dtype == ODY_F32 && D == 64) return launch_delta<float, 64>(p, st);
  if (dtype == ODY_F32 && D == 128) return launch_delta<float, 128>(p, st);
  if (dtype == ODY_BF16 && D == 64) return launch_delta<bf16, 64>(p, st);
  if (dtype == ODY_BF16 && D == 128) return launch_delta<bf16, 128>(p, st);
  ody_set_error("attention: head_dim %d / dtype %d not built", D, dtype);
  return ODY_ERR_UNSUPPORTED;
}
