// Flash-attention backward, head_dim 128, bf16: the dQ kernel on the tile machinery of
// attn_tile.h -- direct global->LDS loads into a three-deep ring, 16-byte LDS reads only
// (K^T comes from the transposed images a pre-pass writes), fenced slots that keep LDS
// operand prefetch and MFMAs interleaved.  Query-stationary, 8 wavefronts x 32 queries
// (two wavefronts per SIMD overlap each other's matrix and vector phases), lane = query
// column, so lse and delta are per-lane scalars:
//
//      S^T = K Q^T            A: K rows (LDS)        B: Q^T (registers)
//      dP^T = V dO^T          A: V rows (LDS)        B: dO^T (registers)
//      dS^T = exp2(S^T c - lse) * (dP^T - delta)
//      dQ^T += K^T dS^T       A: K^T image (LDS)     B: dS^T = accumulator layout
//
// The dK/dV half of the backward is the key-stationary kernel of attn_bwd_mfma.hip.  No
// atomics anywhere: both kernels recompute S, and each owns its outputs.
#include <type_traits>
#include "attn_params.h"
#include "attn_tile.h"

namespace {

using namespace tile128;

constexpr int D = 128, KS = D / 16, DT = D / 32;
#define FENCE() __builtin_amdgcn_sched_barrier(0)

// ---------------------------------------------------------------------------------
// dQ
// ---------------------------------------------------------------------------------
constexpr int DQ_QT = 1, DQ_WAVES = 8, DQ_BM = 32 * DQ_QT * DQ_WAVES, DQ_THREADS = 64 * DQ_WAVES;

__global__ __launch_bounds__(DQ_THREADS) void attn_bwd_dq_pipe_kernel(const AttnParams p,
                                                                       const bf16* __restrict__ kimg) {
  constexpr int BN = 64, QT = DQ_QT;
  constexpr int STAGE = 2 * TILE_ELEMS + IMG_ELEMS;   // K tile, V tile, K^T image
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* ring = reinterpret_cast<bf16*>(smem_raw);     // [3][STAGE]

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 5, i = lane & 31;
  const BlockCoord bc = ody_block_coord(p.Hq, p.B);
  const int nqb = gridDim.x / (p.Hq * p.B);
  const int qblk = p.causal ? (nqb - 1 - bc.rank) : bc.rank;   // heaviest blocks first
  const int h = bc.h, b = bc.b, hk = h / p.group;
  const int q0 = qblk * DQ_BM, wq0 = q0 + wave * 32 * QT;

  const bf16* qp = static_cast<const bf16*>(p.q) + b * p.sq.b + h * p.sq.h;
  const bf16* dop = static_cast<const bf16*>(p.dout) + b * p.sdo.b + h * p.sdo.h;
  const bf16* kp = static_cast<const bf16*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const bf16* vp = static_cast<const bf16*>(p.v) + b * p.sv.b + hk * p.sv.h;
  const int kv_tiles = (p.Lk + BN - 1) / BN;
  const bf16* kip = kimg + ((int64_t)b * p.Hkv + hk) * kv_tiles * IMG_ELEMS;

  const int q_hi = min(q0 + DQ_BM, p.Lq) - 1;
  int n_end = p.causal ? min(p.Lk, q_hi + p.off + 1) : p.Lk;
  if (n_end < 0) n_end = 0;
  const int ntiles = (n_end + BN - 1) / BN;
  int n_full = p.Lk / BN;   // tiles [0, n_full) need no mask for any wavefront of the block
  if (p.causal) n_full = min(n_full, max(0, (q0 + p.off + 1) / BN));
  n_full = min(n_full, ntiles);

  auto load_stage = [&](bf16* st, int t) {
#pragma unroll
    for (int j = 0; j < 16 / DQ_WAVES; j++) {
      const int grp = DQ_WAVES * j + wave;
      int row = t * BN + 4 * grp + (lane & 3);
      row = row < p.Lk ? row : p.Lk - 1;
      const int col = 8 * (lane >> 2);
      __builtin_amdgcn_global_load_lds((global_void_ptr)(kp + (int64_t)row * p.sk.l + col),
                                       (lds_void_ptr)(st + grp * GROUP_ELEMS), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((global_void_ptr)(vp + (int64_t)row * p.sv.l + col),
                                       (lds_void_ptr)(st + TILE_ELEMS + grp * GROUP_ELEMS), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((global_void_ptr)(kip + (int64_t)t * IMG_ELEMS + (grp * 64 + lane) * 8),
                                       (lds_void_ptr)(st + 2 * TILE_ELEMS + grp * 512), 16, 0, 0);
    }
  };
  if (ntiles > 0) load_stage(ring, 0);
  if (ntiles > 1) load_stage(ring + STAGE, 1);

  bf16x8 qf[QT][KS], dof[QT][KS];
  float lse2[QT], delta[QT];
  int lim[QT];
#pragma unroll
  for (int qt = 0; qt < QT; qt++) {
    const int qi = wq0 + 32 * qt + i;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (qi < p.Lq) {
        qf[qt][ks] = *reinterpret_cast<const bf16x8*>(qp + (int64_t)qi * p.sq.l + 16 * ks + 8 * g);
        dof[qt][ks] = *reinterpret_cast<const bf16x8*>(dop + (int64_t)qi * p.sdo.l + 16 * ks + 8 * g);
      } else {
        qf[qt][ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
        dof[qt][ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
    const int64_t ri = ((int64_t)b * p.Hq + h) * p.Lq + qi;
    float l = (qi < p.Lq) ? p.lse[ri] : INFINITY;
    if (l == -INFINITY) l = INFINITY;   // a query that saw no key: P = 0
    lse2[qt] = l * ODY_LOG2E;
    delta[qt] = (qi < p.Lq) ? p.delta[ri] : 0.f;
    lim[qt] = p.causal ? min(p.Lk - 1, qi + p.off) : p.Lk - 1;
  }
  const float c2 = p.scale_log2e;
  const int rbase = row_frag_base(g, i), ibase = image_frag_base(g, i);

  f32x16 dq[QT][DT];
#pragma unroll
  for (int qt = 0; qt < QT; qt++)
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int r = 0; r < 16; r++) dq[qt][dt][r] = 0.f;

  // one 32-key sub-tile x 64 queries: 32 MFMAs for S^T and dP^T, the vector work, 16 MFMAs for
  // dQ^T; every LDS operand fragment feeds two MFMAs
  auto sub_tile = [&](const bf16* st, int t, int kt, bool masked) {
    const bf16* Kt = st + kt * 16;
    const bf16* Vt = st + TILE_ELEMS + kt * 16;
    const bf16* Ki = st + 2 * TILE_ELEMS + kt * 512;
    constexpr int PF = 3;
    bf16x8 kfr[PF], vfr[PF];
#pragma unroll
    for (int n = 0; n < PF; n++) {
      kfr[n] = row_frag(Kt, rbase, n, 0);
      vfr[n] = row_frag(Vt, rbase, n, 0);
    }
    f32x16 s[QT], dp[QT];
    FENCE();
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
#pragma unroll
      for (int qt = 0; qt < QT; qt++) {
        if (ks == 0) {
          s[qt] = mfma32(kfr[0], qf[qt][0], f32x16{0});
          dp[qt] = mfma32(vfr[0], dof[qt][0], f32x16{0});
        } else {
          s[qt] = mfma32(kfr[ks % PF], qf[qt][ks], s[qt]);
          dp[qt] = mfma32(vfr[ks % PF], dof[qt][ks], dp[qt]);
        }
      }
      if (ks + PF < KS) {
        kfr[ks % PF] = row_frag(Kt, rbase, ks + PF, 0);
        vfr[ks % PF] = row_frag(Vt, rbase, ks + PF, 0);
      }
      FENCE();
    }
    bf16x8 ifr[PF];
#pragma unroll
    for (int n = 0; n < PF; n++) ifr[n] = image_frag(Ki, ibase, n & 3, n >> 2, 0);
    if (masked) {
#pragma unroll
      for (int qt = 0; qt < QT; qt++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          if (t * BN + acc_tile_row(r, g, 0) + 2 * kt > lim[qt]) s[qt][r] = -INFINITY;
    }
    bf16x8 dsf[QT][2];
#pragma unroll
    for (int qt = 0; qt < QT; qt++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float pr = ody_exp2(fmaf(s[qt][r], c2, -lse2[qt]));
        dsf[qt][r >> 3][r & 7] = (bf16)(pr * (dp[qt][r] - delta[qt]));
      }
    FENCE();
#pragma unroll
    for (int n = 0; n < 8; n++) {
      const int dt = n & 3, ss = n >> 2;
#pragma unroll
      for (int qt = 0; qt < QT; qt++) dq[qt][dt] = mfma32(ifr[n % PF], dsf[qt][ss], dq[qt][dt]);
      if (n + PF < 8) ifr[n % PF] = image_frag(Ki, ibase, (n + PF) & 3, (n + PF) >> 2, 0);
      FENCE();
    }
  };

  for (int t = 0; t < ntiles; t++) {
    // stage t landed (the loads of stage t+1 may still be in flight), everyone done with stage t-1
    if (t + 1 < ntiles) {
      if (DQ_WAVES == 8) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    }
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (t + 2 < ntiles) load_stage(ring + ((t + 2) % 3) * STAGE, t + 2);
    const bf16* st = ring + (t % 3) * STAGE;
    if (p.causal && t * BN > wq0 + 32 * QT - 1 + p.off) continue;   // every key of the tile is after this wavefront's queries
#pragma unroll 1
    for (int kt = 0; kt < 2; kt++) sub_tile(st, t, kt, t >= n_full);
  }

#pragma unroll
  for (int qt = 0; qt < QT; qt++) {
    const int qi = wq0 + 32 * qt + i;
    if (qi < p.Lq) {
      bf16* dqp = static_cast<bf16*>(p.dq) + b * p.sdq.b + h * p.sdq.h + (int64_t)qi * p.sdq.l;
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int a = 0; a < 4; a++) {
          bf16x4* dst = reinterpret_cast<bf16x4*>(dqp + 32 * dt + 8 * a + 4 * g);
          bf16x4 w, old = {0, 0, 0, 0};
          if (p.accumulate_dq) old = *dst;
#pragma unroll
          for (int e = 0; e < 4; e++) w[e] = (bf16)(dq[qt][dt][4 * a + e] * p.scale + (float)old[e]);
          *dst = w;
        }
    }
  }
}

inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

}  // namespace

// workspace after delta: the transposed images of K
size_t ody_attn_bwd_pipe_workspace(int B, int Lq, int Lk, int Hq, int Hkv) {
  (void)Lq; (void)Hq;
  return align256(ody_attn_images_bytes(B, Lk, Hkv));
}

int ody_launch_attn_bwd_pipe(const AttnParams& p, void* workspace, hipStream_t st) {
  constexpr size_t smem_q = (size_t)3 * (2 * TILE_ELEMS + IMG_ELEMS) * sizeof(bf16);
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_bwd_dq_pipe_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_q) != hipSuccess) {
      ody_set_error("attn_bwd: hipFuncSetAttribute failed");
      return ODY_ERR_LAUNCH;
    }
    attr_set = true;
  }
  bf16* kimg = static_cast<bf16*>(workspace);
  int rc;
  if ((rc = ody_launch_attn_images(p.k, p.sk, p.B, p.Lk, p.Hkv, kimg, nullptr, 0, st))) return rc;
  if ((rc = ody_launch_attn_bwd_dkdv_mfma(p, st))) return rc;
  dim3 gq(((p.Lq + DQ_BM - 1) / DQ_BM) * p.Hq * p.B);
  ODY_LAUNCH("attn_bwd_dq_pipe", st, attn_bwd_dq_pipe_kernel, gq, dim3(DQ_THREADS), smem_q, p, kimg);
  return ody_check_launch("attn_bwd_dq_pipe");
}
