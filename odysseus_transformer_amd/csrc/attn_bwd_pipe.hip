// Flash-attention backward, head_dim 128, bf16, on the tile machinery of attn_tile.h: direct
// global->LDS loads into a ring of stages, 16-byte LDS reads only (an operand that a product
// contracts over its row index comes from the transposed images a pre-pass writes), fenced slots
// that keep LDS operand prefetch and MFMAs interleaved, 8 wavefronts per block = two per SIMD,
// which overlap each other's matrix and vector phases.  Two kernels, no atomics: both recompute S
// from the saved log-sum-exp, and each owns its outputs.
//
// dQ kernel -- query-stationary, 32 queries per wavefront, lane = query column, so lse and delta
// are per-lane scalars; a three-deep ring of {K tile, V tile, K^T image}:
//
//      S^T = K Q^T            A: K rows (LDS)        B: Q^T (registers)
//      dP^T = V dO^T          A: V rows (LDS)        B: dO^T (registers)
//      dS^T = exp2(S^T c - lse) * (dP^T - delta)
//      dQ^T += K^T dS^T       A: K^T image (LDS)     B: dS^T = accumulator layout
//
// dK/dV kernel -- key-stationary, 32 keys per wavefront (described where it is defined).
#include <algorithm>
#include <type_traits>
#include <utility>
#include "attn_params.h"
#include "attn_tile.h"

namespace {

using namespace tile128;

constexpr int D = 128, KS = D / 16, DT = D / 32;
#define FENCE() __builtin_amdgcn_sched_barrier(0)

// dQ^T of one query held by lane group g (accumulator rows 8 (r >> 2) + 4 g + (r & 3) of each 32-wide slice of the
// head dimension) -> row qi of dq: scaled, then added to an fp32 or bf16 destination, rotated back by the rotary
// table, or rounded and stored.
__device__ __forceinline__ void store_dq_row(const AttnParams& p, const f32x16 (&dq)[DT], int b, int h, int qi, int g) {
  if (qi >= p.Lq) return;
  if (p.dq_f32) {
    // fp32 destination (the ring step's running dq): exact accumulation over the key blocks, no rounding here
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
  } else if (p.rope_q) {
    // the gradient of the un-rotated projection: element d < 64 pairs with d + 64, both in this lane
    bf16* dqp = static_cast<bf16*>(p.dq) + b * p.sdq.b + h * p.sdq.h + (int64_t)qi * p.sdq.l;
    const bf16* trow = p.rope_q + ((int64_t)b * p.Lq + qi) * D;
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int a = 0; a < 4; a++) {
        const bf16x8 cs = *reinterpret_cast<const bf16x8*>(trow + 2 * (32 * dt + 8 * a + 4 * g));
        bf16x4 w1, w2;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float c = (float)cs[2 * e], sn = (float)cs[2 * e + 1];
          const float g1 = dq[dt][4 * a + e] * p.scale, g2 = dq[dt + 2][4 * a + e] * p.scale;
          w1[e] = (bf16)(g1 * c + g2 * sn);
          w2[e] = (bf16)(g2 * c - g1 * sn);
        }
        *reinterpret_cast<bf16x4*>(dqp + 32 * dt + 8 * a + 4 * g) = w1;
        *reinterpret_cast<bf16x4*>(dqp + 32 * (dt + 2) + 8 * a + 4 * g) = w2;
      }
  } else {
    bf16* dqp = static_cast<bf16*>(p.dq) + b * p.sdq.b + h * p.sdq.h + (int64_t)qi * p.sdq.l;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int a = 0; a < 4; a++) {
        bf16x4* dst = reinterpret_cast<bf16x4*>(dqp + 32 * dt + 8 * a + 4 * g);
        bf16x4 w, old = {0, 0, 0, 0};
        if (p.accumulate_dq) old = *dst;
#pragma unroll
        for (int e = 0; e < 4; e++) w[e] = (bf16)(dq[dt][4 * a + e] * p.scale + (float)old[e]);
        *dst = w;
      }
  }
}

// The same accumulators as one part's unscaled fp32 sum (a dQ kernel whose key range is cut into parts):
// dq_part [part][B][Lq][Hq][D]; attn_bwd_dq_sum_kernel adds the parts and finishes dq as store_dq_row would.
__device__ __forceinline__ void store_dq_part(float* __restrict__ dq_part, int part, const AttnParams& p,
                                              const f32x16 (&dq)[DT], int b, int h, int qi, int g) {
  if (qi >= p.Lq) return;
  float* dst = dq_part + ((((int64_t)part * p.B + b) * p.Lq + qi) * p.Hq + h) * D;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int a = 0; a < 4; a++) {
      f32x4 w;
#pragma unroll
      for (int e = 0; e < 4; e++) w[e] = dq[dt][4 * a + e];
      *reinterpret_cast<f32x4*>(dst + 32 * dt + 8 * a + 4 * g) = w;
    }
}

// ---------------------------------------------------------------------------------
// dQ
// ---------------------------------------------------------------------------------
constexpr int DQ_QT = 1, DQ_WAVES = 8, DQ_BM = 32 * DQ_QT * DQ_WAVES, DQ_THREADS = 64 * DQ_WAVES;
static_assert(DQ_WAVES == 8, "the load split and the vmcnt waits assume 8 wavefronts");

// kparts > 1 (too few query blocks for the chip): block id = part + kparts * (the usual id), the block takes part
// `part` of its key tiles and leaves its unscaled fp32 sum in dq_part.
__global__ __launch_bounds__(DQ_THREADS) void attn_bwd_dq_pipe_kernel(const AttnParams p,
                                                                       const bf16* __restrict__ kimg, int kparts,
                                                                       float* __restrict__ dq_part) {
  constexpr int BN = 64, QT = DQ_QT;
  constexpr int STAGE = 2 * TILE_ELEMS + IMG_ELEMS;   // K tile, V tile, K^T image
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* ring = reinterpret_cast<bf16*>(smem_raw);     // [3][STAGE]

  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g = lane >> 5,
            i = lane & 31;
  simd_stagger(tid);
  const int kpart = blockIdx.x % kparts;
  const BlockCoord bc = ody_block_coord_of(blockIdx.x / kparts, p.Hq, p.B);
  const int nqb = gridDim.x / (p.Hq * p.B * kparts);
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
  int ntiles = (n_end + BN - 1) / BN;
  int n_full = p.Lk / BN;   // tiles [0, n_full) need no mask for any wavefront of the block
  if (p.causal) n_full = min(n_full, max(0, (q0 + p.off + 1) / BN));
  n_full = min(n_full, ntiles);
  int t_first = 0;   // this block's part of the tiles: [t_first, ntiles)
  if (kparts > 1) {
    const int per = (ntiles + kparts - 1) / kparts;
    t_first = min(kpart * per, ntiles);
    ntiles = min(t_first + per, ntiles);
  }

  auto load_part = [&](bf16* st, int t, int j) {   // j = 0, 1: the two halves of a stage's loads
    {
      const int grp = DQ_WAVES * j + wave;
      int row = t * BN + 4 * grp + (lane >> 4);
      row = row < p.Lk ? row : p.Lk - 1;
      const int col = 8 * (lane & 15);
      __builtin_amdgcn_global_load_lds((global_void_ptr)(kp + (int64_t)row * p.sk.l + col),
                                       (lds_void_ptr)(st + grp * GROUP_ELEMS), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((global_void_ptr)(vp + (int64_t)row * p.sv.l + col),
                                       (lds_void_ptr)(st + TILE_ELEMS + grp * GROUP_ELEMS), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((global_void_ptr)(kip + (int64_t)t * IMG_ELEMS + (grp * 64 + lane) * 8),
                                       (lds_void_ptr)(st + 2 * TILE_ELEMS + grp * 512), 16, 0, 0);
    }
  };
  auto load_stage = [&](bf16* st, int t) {
    load_part(st, t, 0);
    load_part(st, t, 1);
  };
  if (t_first < ntiles) load_stage(ring, t_first);
  if (t_first + 1 < ntiles) load_stage(ring + STAGE, t_first + 1);

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

  // One 64-key tile against this wavefront's 32 queries, as two 32-key sub-tiles kt = 0, 1 with their
  // own accumulation chains: 32 MFMAs for S^T and dP^T, the vector work, 16 MFMAs for dQ^T.
  auto tile = [&](const bf16* st, int t, bool masked) {
    const bf16* Kt = st;
    const bf16* Vt = st + TILE_ELEMS;
    const bf16* Ki = st + 2 * TILE_ELEMS;
    constexpr int PF = 2;
    bf16x8 kfr[PF][2], vfr[PF][2];
#pragma unroll
    for (int n = 0; n < PF; n++)
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
        kfr[n][kt] = row_frag(Kt, rbase, n, kt);
        vfr[n][kt] = row_frag(Vt, rbase, n, kt);
      }
    f32x16 s[2], dp[2];
    FENCE();
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
        if (ks == 0) {
          s[kt] = mfma32(kfr[0][kt], qf[0][0], f32x16{0});
          dp[kt] = mfma32(vfr[0][kt], dof[0][0], f32x16{0});
        } else {
          s[kt] = mfma32(kfr[ks % PF][kt], qf[0][ks], s[kt]);
          dp[kt] = mfma32(vfr[ks % PF][kt], dof[0][ks], dp[kt]);
        }
      }
      if (ks + PF < KS) {
#pragma unroll
        for (int kt = 0; kt < 2; kt++) {
          kfr[ks % PF][kt] = row_frag(Kt, rbase, ks + PF, kt);
          vfr[ks % PF][kt] = row_frag(Vt, rbase, ks + PF, kt);
        }
      }
      FENCE();
    }
    constexpr int IPF = 4;
    bf16x8 ifr[IPF];
#pragma unroll
    for (int n = 0; n < IPF; n++) ifr[n] = image_frag(Ki, ibase, n & 3, 0, 0);
    if (masked) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          if (t * BN + acc_tile_row(r, g, kt) > lim[0]) s[kt][r] = -INFINITY;
    }
    bf16x8 dsf[2][2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float pr = ody_exp2(fmaf(s[kt][r], c2, -lse2[0]));
        dsf[kt][r >> 3][r & 7] = (bf16)(pr * (dp[kt][r] - delta[0]));
      }
    FENCE();
#pragma unroll
    for (int n = 0; n < 16; n++) {
      const int dt = n & 3, ss = (n >> 2) & 1, kt = n >> 3;
      dq[0][dt] = mfma32(ifr[n % IPF], dsf[kt][ss], dq[0][dt]);
      if (n + IPF < 16) {
        const int m = n + IPF;
        ifr[n % IPF] = image_frag(Ki, ibase, m & 3, (m >> 2) & 1, m >> 3);
      }
      FENCE();
    }
  };

  for (int t = t_first; t < ntiles; t++) {
    // stage t landed (the loads of stage t+1 may still be in flight), everyone done with stage t-1
    if (t + 1 < ntiles) {
      asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    } else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const bf16* st = ring + ((t - t_first) % 3) * STAGE;
    const bool dead = p.causal && t * BN > wq0 + 32 * QT - 1 + p.off;   // every key of the tile is after this wavefront's queries
    if (!dead) tile(st, t, t >= n_full);
    // the loads go last: issuing them costs this wavefront time, and here it would otherwise wait at the barrier
    if (t + 2 < ntiles) load_part(ring + ((t + 2 - t_first) % 3) * STAGE, t + 2, 0);
    if (t + 2 < ntiles) load_part(ring + ((t + 2 - t_first) % 3) * STAGE, t + 2, 1);
  }

  if (kparts > 1) store_dq_part(dq_part, kpart, p, dq[0], b, h, wq0 + i, g);
  else store_dq_row(p, dq[0], b, h, wq0 + i, g);
}

// ---------------------------------------------------------------------------------
// dK / dV
// ---------------------------------------------------------------------------------
// Key-stationary, 8 wavefronts x 32 keys (two wavefronts per SIMD), lane = key column.  K and V
// rows stay in registers as B operands; 64-query tiles of Q and dO stream through a two-deep
// ring as row tiles (A operands of S and dP) and as transposed images (A operands of dV^T and
// dK^T); P and dS are accumulator tiles, which is the B-operand layout of the next product.
//
//      S  = Q K^T - lse/scale     the accumulators start at -lse/scale, so P = exp2(S c)
//      dP = dO V^T - delta        likewise -delta
//      dV^T += dO^T P             dK^T += Q^T (P o dP)
constexpr int KV_WAVES = 8, KV_BN = 32 * KV_WAVES, KV_BQ = 64, KV_THREADS = 64 * KV_WAVES;
constexpr int KV_STAT_ELEMS = 64 * 8;                                    // start-value record of one tile: 1 KB, one direct load
constexpr int KV_STAGE = 2 * TILE_ELEMS + 2 * IMG_ELEMS + KV_STAT_ELEMS;   // Q, dO tiles; Q^T, dO^T images; start values

// dS kept for the dQ kernel (Lq and Lk multiples of 256; causal: Lq == Lk): one 128 KB block per (256-key block kb,
// 256-query block qb; causal: qb >= kb), laid out for the reader, which takes 64 keys x 256 queries at a time:
//   [64-key tile y = 0..3][64-query tile x = 0..3][chunk c = 0..7][key 0..63][8 bf16]
// Element j of chunk c is the query of tile row 32 (j >> 2) + 16 (c & 1) + 4 (j & 3) + ((c >> 1) & 1) + 2 (c >> 2) -- the
// order in which an accumulator holds the rows, i.e. image_pos(row) = 8 c + j.  Blocks of one (batch, head) are
// contiguous, key block after key block, and inside a key block by qb.  Entries of masked pairs are 0; the parts
// (y, x) of a diagonal block with y > x, whose keys all come after their queries, are never written (and never used).
constexpr int DS_PIECE = 64 * 8;                 // one (y, x, c): 1 KB
constexpr int DS_PART = 4 * 8 * DS_PIECE;        // one y: 32 KB
constexpr int DS_BLOCK_ELEMS = 4 * DS_PART;
// nbq, nbk: 256-row blocks of queries and of keys.  Causal (nbq == nbk): the blocks at or below the diagonal.
__host__ __device__ inline int64_t ds_blocks_per_head(int nbq, int nbk, bool causal) {
  return causal ? (int64_t)nbq * (nbq + 1) / 2 : (int64_t)nbq * nbk;
}
__host__ __device__ inline int64_t ds_block_index(int nbq, int kb, int qb, bool causal) {
  return causal ? (int64_t)kb * nbq - (int64_t)kb * (kb - 1) / 2 + (qb - kb) : (int64_t)kb * nbq + qb;
}

// S and dP do not start from zero: the accumulators of a sub-tile are loaded with -lse/scale and -delta of their
// rows, so that S comes out of the MFMAs as q.k - lse/scale and P = exp2(S c) costs one multiply and one exp per
// element.  A lane's 16 accumulator rows depend on its lane group only, so the 32 lanes of a group read the same 16
// floats (4 broadcast reads of 16 bytes per product).  The query-side pre-pass (attn_bwd_prepass_kernel) writes them:
// per (batch, head, tile) a table [sub-tile mt][0: -lse/scale, 1: -delta][lane group g][register r] of fp32 at the
// start of a 1 KB record, register r of group g being query acc_tile_row(r, g, mt).  Rows that must give P = 0
// (beyond Lq, or a query that saw no key) hold -1e30.
//
// SPLIT = false: a block owns 256 keys of one kv head and walks all query heads of its group.
// SPLIT = true (grouped-query attention, or too few key blocks for the chip): a block owns 256 keys for ONE query
// head and part `bc.h % qparts` of that head's query tiles, and writes fp32 partial dK / dV to `part`, which
// attn_bwd_group_sum_kernel adds up over the group and the parts.  With few kv heads, or few keys against many
// queries (a ring step over a short key block), this is what gives the chip enough, and evenly sized, blocks.
//
// KEEP_DS = true (whole 256-row blocks on both sides; causal: self-attention): every dS tile also goes to p.ds, in the
// layout described at ds_block_index, and the dQ kernel below (attn_bwd_dq_kept_kernel) reads it back
// instead of computing S, dP and dS a second time.
template <bool SPLIT, bool KEEP_DS>
__global__ __launch_bounds__(KV_THREADS) void attn_bwd_dkdv_pipe_kernel(const AttnParams p,
                                                                         const bf16* __restrict__ qimg,
                                                                         const bf16* __restrict__ doimg,
                                                                         const bf16* __restrict__ stats,
                                                                         float* __restrict__ part, int qparts) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* ring = reinterpret_cast<bf16*>(smem_raw);   // [2][KV_STAGE]

  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g = lane >> 5,
            i = lane & 31;
  const BlockCoord bc = ody_block_coord(SPLIT ? p.Hq * qparts : p.Hkv, p.B);   // rank 0 = first key block = most query tiles
  const int hq = SPLIT ? bc.h / qparts : 0, qpart = SPLIT ? bc.h % qparts : 0;
  const int hk = SPLIT ? hq / p.group : bc.h, b = bc.b;
  const int h_first = SPLIT ? hq : hk * p.group, n_heads = SPLIT ? 1 : p.group;   // query heads this block walks
  const int n0 = bc.rank * KV_BN, wn0 = n0 + wave * 32, key = wn0 + i;
  const int q_tiles = (p.Lq + KV_BQ - 1) / KV_BQ;
  simd_stagger(tid);

  bf16x8 kf[KS], vf[KS];
  {
    const bf16* kp = static_cast<const bf16*>(p.k) + b * p.sk.b + hk * p.sk.h;
    const bf16* vp = static_cast<const bf16*>(p.v) + b * p.sv.b + hk * p.sv.h;
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
  }
  f32x16 dk[DT], dv[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) dk[dt][r] = dv[dt][r] = 0.f;

  const int t_begin = p.causal ? max(0, n0 - p.off) / KV_BQ : 0;   // first query tile that sees a key of this block
  int ntq = max(0, q_tiles - t_begin), t_top = q_tiles - 1;   // this block's tiles: t_top, t_top - 1, ... (ntq of them)
  if (SPLIT && qparts > 1) {
    const int per = (ntq + qparts - 1) / qparts;
    t_top -= qpart * per;
    ntq = max(0, min(per, ntq - qpart * per));
  }
  const int total = ntq * n_heads;   // flattened (query head, query tile)
  const float c2 = p.scale_log2e;

  // Direct loads of one stage: uniform base pointers plus 32-bit per-lane offsets that are
  // recomputed from the lane id every time (cheaper than keeping them in registers here).
  auto load_stage = [&](bf16* st, int it, int j) {   // j = 0, 1: the two halves of the stage's loads
    const int hg = it / ntq, t = t_top - (it % ntq), h = h_first + hg;
    const bf16* qp = static_cast<const bf16*>(p.q) + b * p.sq.b + h * p.sq.h + (int64_t)t * KV_BQ * p.sq.l;
    const bf16* dop = static_cast<const bf16*>(p.dout) + b * p.sdo.b + h * p.sdo.h + (int64_t)t * KV_BQ * p.sdo.l;
    const int64_t tile_id = ((int64_t)b * p.Hq + h) * q_tiles + t;
    const bf16* qi_ = qimg + tile_id * IMG_ELEMS;
    const bf16* doi = doimg + tile_id * IMG_ELEMS;
    const int rmax = p.Lq - 1 - t * KV_BQ;   // rows beyond the matrix re-read its last row
    const int ln = fresh_lane();
    if (j == 0 && wave == KV_WAVES - 1)
      __builtin_amdgcn_global_load_lds((global_void_ptr)(stats + tile_id * KV_STAT_ELEMS + (unsigned)(ln * 8)),
                                       (lds_void_ptr)(st + 2 * TILE_ELEMS + 2 * IMG_ELEMS), 16, 0, 0);
    {
      const int grp = KV_WAVES * j + wave;
      const int row = min(4 * grp + (ln >> 4), rmax), col = 8 * (ln & 15);
      __builtin_amdgcn_global_load_lds((global_void_ptr)(qp + (unsigned)(row * (int)p.sq.l + col)),
                                       (lds_void_ptr)(st + grp * GROUP_ELEMS), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((global_void_ptr)(dop + (unsigned)(row * (int)p.sdo.l + col)),
                                       (lds_void_ptr)(st + TILE_ELEMS + grp * GROUP_ELEMS), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((global_void_ptr)(qi_ + (unsigned)((grp * 64 + ln) * 8)),
                                       (lds_void_ptr)(st + 2 * TILE_ELEMS + grp * 512), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((global_void_ptr)(doi + (unsigned)((grp * 64 + ln) * 8)),
                                       (lds_void_ptr)(st + 2 * TILE_ELEMS + IMG_ELEMS + grp * 512), 16, 0, 0);
    }
  };
  if (total > 0) {
    load_stage(ring, 0, 0);
    load_stage(ring, 0, 1);
  }

  // one 32-query sub-tile against this wavefront's 32 keys: 16 MFMAs for S and dP on top of their
  // start values, the vector work, 16 MFMAs for dV^T and dK^T
  // kept dS: chunk 4 mt + 2 ss + g of part (y, x) = (wave >> 1, t & 3) of the block, to which `tile` points at this
  // wavefront's 32 keys.  Streaming stores: the tiles are read once, by another kernel.
  auto sub_tile = [&](const bf16* st, int t, int mt, bool masked, bf16* ds_tile) {
    const int ln = fresh_lane(), g = ln >> 5, i = ln & 31;
    const int rbase = row_frag_base(g, i), ibase = image_frag_base(g, i);
    const bf16* Qt = st;
    const bf16* Ot = st + TILE_ELEMS;
    const bf16* Qi = st + 2 * TILE_ELEMS;
    const bf16* Oi = Qi + IMG_ELEMS;
    constexpr int PF = 2;
    bf16x8 qfr[PF], ofr[PF];
    f32x16 s, dp;
    {
      const float* Sf = reinterpret_cast<const float*>(Oi + IMG_ELEMS) + mt * 64 + g * 16;
#pragma unroll
      for (int a = 0; a < 4; a++) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(Sf + 4 * a), w = *reinterpret_cast<const f32x4*>(Sf + 32 + 4 * a);
#pragma unroll
        for (int e = 0; e < 4; e++) s[4 * a + e] = v[e], dp[4 * a + e] = w[e];
      }
    }
    qfr[0] = row_frag(Qt, rbase, 0, mt);
    ofr[0] = row_frag(Ot, rbase, 0, mt);
    qfr[1] = row_frag(Qt, rbase, 1, mt);
    ofr[1] = row_frag(Ot, rbase, 1, mt);
    FENCE();
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      s = mfma32(qfr[ks % PF], kf[ks], s);
      dp = mfma32(ofr[ks % PF], vf[ks], dp);
      if (ks + PF < KS) {
        qfr[ks % PF] = row_frag(Qt, rbase, ks + PF, mt);
        ofr[ks % PF] = row_frag(Ot, rbase, ks + PF, mt);
      }
      FENCE();
    }
    bf16x8 oif[PF], qif[PF];
#pragma unroll
    for (int n = 0; n < PF; n++) {
      oif[n] = image_frag(Oi, ibase, n & 3, n >> 2, mt);
      qif[n] = image_frag(Qi, ibase, n & 3, n >> 2, mt);
    }
    if (masked) {
      const int lim = wn0 + i - p.off - t * KV_BQ;   // tile rows below lim come before this lane's key
#pragma unroll
      for (int r = 0; r < 16; r++)
        if (acc_tile_row(r, g, mt) < lim) s[r] = -INFINITY;
    }
    bf16x8 pf[2], dsf[2];
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const float pr = ody_exp2(s[r] * c2);
      pf[r >> 3][r & 7] = (bf16)pr;
      dsf[r >> 3][r & 7] = (bf16)(pr * dp[r]);
    }
    // Kept dS: dsf[ss] is chunk 4 mt + 2 ss + g of this lane's key, 512 contiguous bytes per half wavefront;
    // ds_tile points at part (y, x) = (wave >> 1, t & 3) of the block, at this wavefront's 32 keys.  Streaming
    // stores (the tiles are read once, by another kernel), one under each half of the MFMAs below.  (Holding them
    // back in LDS until the next sub-tile, so that none is still on its way at the top of the next iteration, where
    // the wait for the tile loads waits for stores as well, was measured slower.)
    auto keep = [&](int ss) {
      typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
      u32x4* dst = reinterpret_cast<u32x4*>(ds_tile + (unsigned)((4 * mt + 2 * ss + g) * DS_PIECE + i * 8));
      __builtin_nontemporal_store(__builtin_bit_cast(u32x4, dsf[ss]), dst);
    };
    FENCE();
#pragma unroll
    for (int n = 0; n < 8; n++) {
      const int dt = n & 3, ss = n >> 2;
      if (KEEP_DS && (n == 1 || n == 5)) keep(n >> 2);
      dv[dt] = mfma32(oif[n % PF], pf[ss], dv[dt]);
      dk[dt] = mfma32(qif[n % PF], dsf[ss], dk[dt]);
      if (n + PF < 8) {
        oif[n % PF] = image_frag(Oi, ibase, (n + PF) & 3, (n + PF) >> 2, mt);
        qif[n % PF] = image_frag(Qi, ibase, (n + PF) & 3, (n + PF) >> 2, mt);
      }
      FENCE();
    }
  };

  for (int it = 0; it < total; it++) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int t = t_top - (it % ntq);   // last query tile first: the key blocks of an XCD then read the same
                                              // Q / dO tiles at the same time and share them through L2
    const bf16* st = ring + (it & 1) * KV_STAGE;
    // every query of the tile is before every key of this wavefront: nothing to do
    const bool dead = p.causal && (t * KV_BQ + KV_BQ - 1 + p.off < wn0);
    const bool masked = p.causal && (t * KV_BQ + p.off < wn0 + 31);
    bf16* ds_tile = nullptr;
    if (KEEP_DS) {
      const int nbq = q_tiles / 4, nbk = p.Lk / KV_BN;
      ds_tile = p.ds + (((int64_t)b * p.Hq + h_first + it / ntq) * ds_blocks_per_head(nbq, nbk, p.causal) +
                        ds_block_index(nbq, bc.rank, t >> 2, p.causal)) * DS_BLOCK_ELEMS +
                (((wave >> 1) * 4 + (t & 3)) * 8) * DS_PIECE + (wave & 1) * 32 * 8;
    }
#pragma unroll 1
    for (int mt = 0; mt < 2; mt++) {
      // the loads of the next stage go out in two halves, one before each sub-tile: issued all at
      // once by eight wavefronts they would queue up behind each other at the memory pipeline
      if (it + 1 < total) load_stage(ring + ((it + 1) & 1) * KV_STAGE, it + 1, mt);
      if (!dead) sub_tile(st, t, mt, masked, ds_tile);
    }
  }

  if (SPLIT) {
    if (key < p.Lk) {
      // part: [dK | dV][batch][query head][part of the queries][key][D] fp32, unscaled
      float* pk = part + (((int64_t)b * p.Hq * qparts + bc.h) * p.Lk + key) * D;
      float* pv = pk + (int64_t)p.B * p.Hq * qparts * p.Lk * D;
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int a = 0; a < 4; a++) {
          f32x4 wk, wv;
#pragma unroll
          for (int e = 0; e < 4; e++) wk[e] = dk[dt][4 * a + e], wv[e] = dv[dt][4 * a + e];
          *reinterpret_cast<f32x4*>(pk + 32 * dt + 8 * a + 4 * g) = wk;
          *reinterpret_cast<f32x4*>(pv + 32 * dt + 8 * a + 4 * g) = wv;
        }
    }
  } else if (key < p.Lk) {
    bf16* dkp = static_cast<bf16*>(p.dk) + b * p.sdk.b + hk * p.sdk.h + (int64_t)key * p.sdk.l;
    bf16* dvp = static_cast<bf16*>(p.dv) + b * p.sdv.b + hk * p.sdv.h + (int64_t)key * p.sdv.l;
    const bf16* trow = p.rope_k ? p.rope_k + ((int64_t)b * p.Lk + key) * D : nullptr;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int a = 0; a < 4; a++) {
        bf16x4 wv;
#pragma unroll
        for (int e = 0; e < 4; e++) wv[e] = (bf16)dv[dt][4 * a + e];
        *reinterpret_cast<bf16x4*>(dvp + 32 * dt + 8 * a + 4 * g) = wv;
      }
    if (trow) {   // dK of the un-rotated projection: element d < 64 pairs with d + 64, both in this lane
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int a = 0; a < 4; a++) {
          const bf16x8 cs = *reinterpret_cast<const bf16x8*>(trow + 2 * (32 * dt + 8 * a + 4 * g));
          bf16x4 w1, w2;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float c = (float)cs[2 * e], sn = (float)cs[2 * e + 1];
            const float g1 = dk[dt][4 * a + e] * p.scale, g2 = dk[dt + 2][4 * a + e] * p.scale;
            w1[e] = (bf16)(g1 * c + g2 * sn);
            w2[e] = (bf16)(g2 * c - g1 * sn);
          }
          *reinterpret_cast<bf16x4*>(dkp + 32 * dt + 8 * a + 4 * g) = w1;
          *reinterpret_cast<bf16x4*>(dkp + 32 * (dt + 2) + 8 * a + 4 * g) = w2;
        }
    } else {
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int a = 0; a < 4; a++) {
          bf16x4 wk;
#pragma unroll
          for (int e = 0; e < 4; e++) wk[e] = (bf16)(dk[dt][4 * a + e] * p.scale);
          *reinterpret_cast<bf16x4*>(dkp + 32 * dt + 8 * a + 4 * g) = wk;
        }
    }
  }
}

// ---------------------------------------------------------------------------------
// dQ from the kept dS
// ---------------------------------------------------------------------------------
// One product, dQ^T += K^T dS^T, over the tiles that the dK/dV kernel (KEEP_DS) left in p.ds.  256 queries per block,
// 8 wavefronts x 32 queries: wavefront w owns chunks 4 (w & 1) ... + 3 of 64-query tile (w >> 1) of the block, lane i
// the query at position 32 (w & 1) + i of that tile's kept order.
//
//      A: K^T image (LDS, 16-byte reads), as in the dQ kernel at the top of this file
//      B: dS^T.  The tiles hold 8 queries of one key side by side, the product contracts over keys: the transposing
//         LDS read turns 4 keys x 16 queries into 4-key pieces per query, two of them make a fragment.
//
// 2 bytes per visible (query, key) pair for 256 flops: the kernel is bound by HBM, and what it needs is bytes in
// flight -- more than the LDS could take as landing room.  So the dS of a 64-key tile (32 one-KB pieces, 4 per
// wavefront) and its K^T image (2 KB per wavefront) travel through registers: four sets, loaded four tiles ahead,
// written to one of two LDS buffers the iteration before their tile is due.  (Direct loads to LDS for the images
// would put two kinds of loads on the one counter, and the compiler then waits for all of them every time.)
// The compiler places the waits for the register loads by counting the loads issued since, so these must leave in
// program order: no pass may move a load across this point, neither the optimizer nor the instruction scheduler.
#define ISSUE_ORDER()                    \
  do {                                   \
    asm volatile("" ::: "memory");       \
    __builtin_amdgcn_sched_barrier(0);   \
  } while (0)
constexpr int DS_PIECE_ELEMS = GROUP_ELEMS;   // 1 KB + 16 bytes: consecutive pieces start 4 banks apart
constexpr int DQK_DS_BUF = 32 * DS_PIECE_ELEMS, DQK_SETS = 4;
constexpr int DQK_LDS_ELEMS = 2 * DQK_DS_BUF + 2 * IMG_ELEMS;

//
// kparts > 1 (too few query blocks for the chip: a ring step of few queries against a long key block): block id =
// part + kparts * (the usual id), the block takes part `part` of its 256-key blocks and leaves its unscaled fp32 sum in
// dq_part [part][B][Lq][Hq][D]; attn_bwd_dq_sum_kernel adds the parts and finishes dq.
__global__ __launch_bounds__(DQ_THREADS) void attn_bwd_dq_kept_kernel(const AttnParams p, const bf16* __restrict__ kimg,
                                                                       int kparts, float* __restrict__ dq_part) {
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* dsbuf = reinterpret_cast<bf16*>(smem_raw);   // [2][DQK_DS_BUF]
  bf16* imgs = dsbuf + 2 * DQK_DS_BUF;               // [2][IMG_ELEMS]

  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g = lane >> 5,
            i = lane & 31;
  const int kpart = blockIdx.x % kparts;
  const BlockCoord bc = ody_block_coord_of(blockIdx.x / kparts, p.Hq, p.B);
  const int nqb = gridDim.x / (p.Hq * p.B * kparts);
  const int qblk = p.causal ? nqb - 1 - bc.rank : bc.rank;   // causal: heaviest blocks first
  const int h = bc.h, b = bc.b, hk = h / p.group;
  const int x = wave >> 1, mt = wave & 1, nbq = p.Lq / KV_BN, nbk = p.Lk / KV_BN;
  const bf16* kip = kimg + ((int64_t)b * p.Hkv + hk) * (p.Lk / 64) * IMG_ELEMS;
  const bf16* dsh = p.ds + ((int64_t)b * p.Hq + h) * ds_blocks_per_head(nbq, nbk, p.causal) * DS_BLOCK_ELEMS;
  // 64-key tiles: all of them, or (causal) those up to the block's last query; a multiple of DQK_SETS
  int ntiles = p.causal ? 4 * (qblk + 1) : 4 * nbk;
  const int last_tile = p.causal ? 4 * qblk + x : ntiles;   // of this wavefront's queries
  int t_first = 0;   // this block's part of the tiles: [t_first, ntiles), whole 256-key blocks
  if (kparts > 1) {
    const int per = 4 * ((ntiles / 4 + kparts - 1) / kparts);
    t_first = min(kpart * per, ntiles);
    ntiles = min(t_first + per, ntiles);
  }
  // position 32 mt + i of the tile's kept order = chunk 4 mt + (i >> 3), element i & 7
  const int qrow = qblk * DQ_BM + KV_BQ * x + 32 * ((i >> 2) & 1) + 16 * ((i >> 3) & 1) + 4 * (i & 3) + (i >> 4) + 2 * mt;
  auto store_part = [&](const f32x16 (&acc)[DT]) { store_dq_part(dq_part, kpart, p, acc, b, h, qrow, g); };

  u32x4 regs[DQK_SETS][6];
  // tile t: this wavefront's 4 of the 32 pieces (x, c) of key tile t & 3 of block (t >> 2, qblk) -- 32 KB in a row --
  // and its 2 of the 16 KB of the K^T image, into register set `set`
  auto issue = [&](int set, int t) {
    const bf16* src = dsh + ds_block_index(nbq, t >> 2, qblk, p.causal) * DS_BLOCK_ELEMS + (t & 3) * DS_PART;
#pragma unroll
    for (int n = 0; n < 4; n++) {   // piece 8 n + wave: query tile n of the block, chunk `wave`
      regs[set][n] = *reinterpret_cast<const u32x4*>(src + (unsigned)((8 * n + wave) * DS_PIECE + lane * 8));
      ISSUE_ORDER();
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
      regs[set][4 + j] = *reinterpret_cast<const u32x4*>(kip + (int64_t)t * IMG_ELEMS + (unsigned)(((DQ_WAVES * j + wave) * 64 + lane) * 8));
      ISSUE_ORDER();
    }
  };
  auto drain = [&](int set, int t) {
    bf16* buf = dsbuf + (t & 1) * DQK_DS_BUF;
#pragma unroll
    for (int n = 0; n < 4; n++)
      *reinterpret_cast<u32x4*>(buf + (8 * n + wave) * DS_PIECE_ELEMS + lane * 8) = regs[set][n];
    bf16* slot = imgs + (t & 1) * IMG_ELEMS;
#pragma unroll
    for (int j = 0; j < 2; j++)
      *reinterpret_cast<u32x4*>(slot + ((DQ_WAVES * j + wave) * 64 + lane) * 8) = regs[set][4 + j];
  };
  f32x16 dq[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq[dt][r] = 0.f;
  if (t_first >= ntiles) {   // a part without keys (causal: an early query block has fewer key blocks than parts)
    store_part(dq);
    return;
  }
#pragma unroll
  for (int u = 0; u < DQK_SETS; u++) issue(u, t_first + u);   // ntiles - t_first >= DQK_SETS

  const int ibase = image_frag_base(g, i);
  // the transposing read: inside 16 lanes, lane 4 k + m supplies key 4 k (+ the fragment's row offset) and queries
  // 4 m ... 4 m + 3 of the 16; queries 0-7 of the 16 are one chunk, 8-15 the next
  const int sbase = (8 * x + 4 * mt + 2 * ((lane >> 4) & 1) + ((lane >> 1) & 1)) * DS_PIECE_ELEMS +
                    (16 * g + 4 * ((lane >> 2) & 3)) * 8 + 4 * (lane & 1);

  auto tile = [&](int t) {
    const bf16* Sp = dsbuf + (t & 1) * DQK_DS_BUF + sbase;
    const bf16* Ki = imgs + (t & 1) * IMG_ELEMS;
    constexpr int IPF = 4;
    bf16x8 ifr[IPF], dsf[2][2];
#pragma unroll
    for (int n = 0; n < IPF; n++) ifr[n] = image_frag(Ki, ibase, n & 3, 0, 0);
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int ss = 0; ss < 2; ss++)   // keys 32 (j >> 2) + 16 g + 4 (j & 3) + ss + 2 kt, j = 0..7
        dsf[kt][ss] = concat4(lds_read_tr16(Sp + (ss + 2 * kt) * 8), lds_read_tr16(Sp + (ss + 2 * kt) * 8 + 32 * 8));
    FENCE();
#pragma unroll
    for (int n = 0; n < 16; n++) {
      const int dt = n & 3, ss = (n >> 2) & 1, kt = n >> 3;
      dq[dt] = mfma32(ifr[n % IPF], dsf[kt][ss], dq[dt]);
      if (n + IPF < 16) {
        const int m = n + IPF;
        ifr[n % IPF] = image_frag(Ki, ibase, m & 3, (m >> 2) & 1, m >> 3);
      }
      FENCE();
    }
  };

  drain(0, t_first);
  ISSUE_ORDER();
  int t0 = t_first;
  do {   // not a `for`: its entry test would give the compiler a block to sink the loads above into, out of order
#pragma unroll
    for (int u = 0; u < DQK_SETS; u++) {
      const int t = t0 + u;
      // everyone is done with tile t - 1, and sees what the wavefronts wrote of tile t to LDS an iteration ago
      __syncthreads();
      // tile t + 1 has arrived (the compiler places the wait: all loads are of one kind, so it can count them);
      // tiles t + 2 and t + 3 may still be on their way, and tile t + 4 sets out
      // No branches around these (past the end: a write that nobody reads, and one more load of the last tile):
      // with branches the compiler loses count of the loads in flight and waits for all of them.
      ISSUE_ORDER();
      drain((u + 1) % DQK_SETS, t + 1);
      ISSUE_ORDER();
      issue(u, min(t + DQK_SETS, ntiles - 1));
      // (causal) tiles whose keys all come after this wavefront's queries were never written
      if (t <= last_tile) tile(t);
    }
  } while ((t0 += DQK_SETS) < ntiles);

  if (kparts > 1) store_part(dq);
  else store_dq_row(p, dq, b, h, qrow, g);
}

// dq = the sum of the fp32 parts of a key-split dQ kernel, finished like store_dq_row does; one thread per
// 4 elements d..d+3 of the first half of a (query, head) row and their partners d + 64 (the pairs of the rotary
// embedding)
__global__ __launch_bounds__(256) void attn_bwd_dq_sum_kernel(const AttnParams p, const float* __restrict__ dq_part, int kparts) {
  constexpr int Q = D / 8;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;   // over B * Lq * Hq * D / 8
  const int64_t total = (int64_t)p.B * p.Lq * p.Hq * Q;
  if (idx >= total) return;
  const int d4 = idx % Q;
  const int h = (idx / Q) % p.Hq;
  const int qi = (idx / ((int64_t)Q * p.Hq)) % p.Lq;
  const int b = idx / ((int64_t)Q * p.Hq * p.Lq);
  const int64_t plane = (int64_t)p.B * p.Lq * p.Hq * D;
  const float* src = dq_part + (((int64_t)b * p.Lq + qi) * p.Hq + h) * D + 4 * d4;
  f32x4 s1 = {0.f, 0.f, 0.f, 0.f}, s2 = s1;
  for (int s = 0; s < kparts; s++) {
    s1 += *reinterpret_cast<const f32x4*>(src + s * plane);
    s2 += *reinterpret_cast<const f32x4*>(src + s * plane + D / 2);
  }
  s1 *= p.scale;
  s2 *= p.scale;
  if (p.dq_f32) {
    float* dqp = static_cast<float*>(p.dq) + b * p.sdq.b + h * p.sdq.h + (int64_t)qi * p.sdq.l + 4 * d4;
    if (p.accumulate_dq) {
      s1 += *reinterpret_cast<const f32x4*>(dqp);
      s2 += *reinterpret_cast<const f32x4*>(dqp + D / 2);
    }
    *reinterpret_cast<f32x4*>(dqp) = s1;
    *reinterpret_cast<f32x4*>(dqp + D / 2) = s2;
    return;
  }
  bf16* dqp = static_cast<bf16*>(p.dq) + b * p.sdq.b + h * p.sdq.h + (int64_t)qi * p.sdq.l + 4 * d4;
  bf16x4 w1, w2;
  if (p.rope_q) {
    const bf16x8 cs = *reinterpret_cast<const bf16x8*>(p.rope_q + ((int64_t)b * p.Lq + qi) * D + 8 * d4);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float c = (float)cs[2 * e], sn = (float)cs[2 * e + 1];
      w1[e] = (bf16)(s1[e] * c + s2[e] * sn);
      w2[e] = (bf16)(s2[e] * c - s1[e] * sn);
    }
  } else {
    if (p.accumulate_dq) {
      const bf16x4 o1 = *reinterpret_cast<const bf16x4*>(dqp), o2 = *reinterpret_cast<const bf16x4*>(dqp + D / 2);
#pragma unroll
      for (int e = 0; e < 4; e++) s1[e] += (float)o1[e], s2[e] += (float)o2[e];
    }
#pragma unroll
    for (int e = 0; e < 4; e++) w1[e] = (bf16)s1[e], w2[e] = (bf16)s2[e];
  }
  *reinterpret_cast<bf16x4*>(dqp) = w1;
  *reinterpret_cast<bf16x4*>(dqp + D / 2) = w2;
}

// dK, dV of a kv head = sum of the fp32 partials of its query heads and their `qparts` parts; one thread per 4 elements
// d..d+3 of the first half of a key row and their partners d + 64 (the pairs of the rotary embedding)
__global__ __launch_bounds__(256) void attn_bwd_group_sum_kernel(const AttnParams p, const float* __restrict__ part,
                                                                 int qparts) {
  constexpr int Q = D / 8;                                                // threads per key row
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;           // over B * Hkv * Lk * D / 8
  const int64_t total = (int64_t)p.B * p.Hkv * p.Lk * Q;
  if (idx >= total) return;
  const int d4 = idx % Q;
  const int key = (idx / Q) % p.Lk;
  const int hk = (idx / ((int64_t)Q * p.Lk)) % p.Hkv;
  const int b = idx / ((int64_t)Q * p.Lk * p.Hkv);
  const int64_t plane = (int64_t)p.B * p.Hq * qparts * p.Lk * D;
  f32x4 sk1 = {0.f, 0.f, 0.f, 0.f}, sk2 = sk1, sv1 = sk1, sv2 = sk1;
  for (int hg = 0; hg < p.group * qparts; hg++) {   // (query head of the group, part), in this fixed order
    const float* src = part + ((((int64_t)b * p.Hkv + hk) * p.group * qparts + hg) * p.Lk + key) * D + 4 * d4;
    sk1 += *reinterpret_cast<const f32x4*>(src);
    sk2 += *reinterpret_cast<const f32x4*>(src + D / 2);
    sv1 += *reinterpret_cast<const f32x4*>(src + plane);
    sv2 += *reinterpret_cast<const f32x4*>(src + plane + D / 2);
  }
  bf16x4 wk1, wk2, wv1, wv2;
  if (p.rope_k) {
    const bf16x8 cs = *reinterpret_cast<const bf16x8*>(p.rope_k + ((int64_t)b * p.Lk + key) * D + 8 * d4);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float c = (float)cs[2 * e], sn = (float)cs[2 * e + 1];
      const float g1 = sk1[e] * p.scale, g2 = sk2[e] * p.scale;
      wk1[e] = (bf16)(g1 * c + g2 * sn);
      wk2[e] = (bf16)(g2 * c - g1 * sn);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; e++) wk1[e] = (bf16)(sk1[e] * p.scale), wk2[e] = (bf16)(sk2[e] * p.scale);
  }
#pragma unroll
  for (int e = 0; e < 4; e++) wv1[e] = (bf16)sv1[e], wv2[e] = (bf16)sv2[e];
  bf16* dkp = static_cast<bf16*>(p.dk) + b * p.sdk.b + hk * p.sdk.h + (int64_t)key * p.sdk.l + 4 * d4;
  bf16* dvp = static_cast<bf16*>(p.dv) + b * p.sdv.b + hk * p.sdv.h + (int64_t)key * p.sdv.l + 4 * d4;
  *reinterpret_cast<bf16x4*>(dkp) = wk1;
  *reinterpret_cast<bf16x4*>(dkp + D / 2) = wk2;
  *reinterpret_cast<bf16x4*>(dvp) = wv1;
  *reinterpret_cast<bf16x4*>(dvp + D / 2) = wv2;
}

inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

// Parts of the other side's range, for a kernel with `blocks` blocks that each walk `tiles` 64-row tiles.  As for the
// forward's key split: with fewer blocks than it takes to keep the chip's 256 compute units busy and balanced -- one
// block each when all are equally long, two each under a causal mask, where they are not and only a second, lighter
// block per unit lets the heaviest-first order even that out -- the range is cut into 2 or 4 parts of at least 16
// tiles (on average, when causal).
inline int range_parts(int64_t blocks, int tiles, bool causal) {
  const int64_t want = causal ? 512 : 256;
  int s = 1;
  while (s < 4 && blocks * s * 2 <= want && tiles >= 32 * s) s *= 2;
  return s;
}
// dK/dV: parts of the query range of a (256-key block, query head)
inline int query_parts(int B, int Lq, int Lk, int Hq, int Hkv, bool causal) {
  const int64_t blocks = (int64_t)B * Hq * ((Lk + KV_BN - 1) / KV_BN);   // already one per QUERY head when they are split
  return range_parts(blocks, (Lq + KV_BQ - 1) / KV_BQ, causal);
}
// dQ (either kernel): parts of the key range of a (256-query block, head)
inline int key_parts(int B, int Lq, int Lk, int Hq, bool causal) {
  return range_parts((int64_t)B * Hq * ((Lq + DQ_BM - 1) / DQ_BM), (Lk + 63) / 64, causal);
}
// fp32 partial dK / dV (grouped-query attention, or a split query range) and partial dQ (a split key range) share one
// region: the first is summed up before the second is written.  Sized for the larger of the causal and the unmasked
// policy, since the size query does not know the mask.
inline size_t partials_bytes(int B, int Lq, int Lk, int Hq, int Hkv) {
  const int qp = std::max(query_parts(B, Lq, Lk, Hq, Hkv, false), query_parts(B, Lq, Lk, Hq, Hkv, true));
  const int kp = std::max(key_parts(B, Lq, Lk, Hq, false), key_parts(B, Lq, Lk, Hq, true));
  const size_t kv = (Hq == Hkv && qp == 1) ? 0 : (size_t)2 * B * Hq * qp * Lk * D * sizeof(float);
  const size_t dq = kp == 1 ? 0 : (size_t)kp * B * Lq * Hq * D * sizeof(float);
  return align256(std::max(kv, dq));
}

}  // namespace

// workspace after delta: the transposed images of K, Q and dO, the per-tile start values and, for
// grouped-query attention, the fp32 partial dK / dV of every query head
size_t ody_attn_bwd_pipe_workspace(int B, int Lq, int Lk, int Hq, int Hkv) {
  return align256(ody_attn_images_bytes(B, Lk, Hkv)) + 2 * align256(ody_attn_images_bytes(B, Lq, Hq)) +
         align256((size_t)B * Hq * ((Lq + KV_BQ - 1) / KV_BQ) * KV_STAT_ELEMS * sizeof(bf16)) +
         partials_bytes(B, Lq, Lk, Hq, Hkv);
}

size_t ody_attn_bwd_pipe_ds_bytes(int B, int Lq, int Lk, int Hq, int causal) {
  if (Lq % KV_BN != 0 || Lk % KV_BN != 0 || (causal && Lq != Lk) || B <= 0 || Hq <= 0) return 0;
  return (size_t)B * Hq * ds_blocks_per_head(Lq / KV_BN, Lk / KV_BN, causal != 0) * DS_BLOCK_ELEMS * sizeof(bf16);
}

int ody_launch_attn_bwd_pipe(const AttnParams& p, void* workspace, hipStream_t st) {
  constexpr size_t smem_q = (size_t)3 * (2 * TILE_ELEMS + IMG_ELEMS) * sizeof(bf16);
  constexpr size_t smem_kv = (size_t)2 * KV_STAGE * sizeof(bf16);
  constexpr size_t smem_qs = (size_t)DQK_LDS_ELEMS * sizeof(bf16);
  static_assert(smem_qs <= 160 * 1024, "LDS of one CU");
  for (const auto& ks : {std::pair<const void*, size_t>{reinterpret_cast<const void*>(&attn_bwd_dq_pipe_kernel), smem_q},
                         {reinterpret_cast<const void*>(&attn_bwd_dq_kept_kernel), smem_qs},
                         {reinterpret_cast<const void*>(&attn_bwd_dkdv_pipe_kernel<false, false>), smem_kv},
                         {reinterpret_cast<const void*>(&attn_bwd_dkdv_pipe_kernel<true, false>), smem_kv},
                         {reinterpret_cast<const void*>(&attn_bwd_dkdv_pipe_kernel<false, true>), smem_kv},
                         {reinterpret_cast<const void*>(&attn_bwd_dkdv_pipe_kernel<true, true>), smem_kv}})
    if (int rc = ody_allow_dynamic_lds(ks.first, ks.second, "attn_bwd")) return rc;
  unsigned char* w = static_cast<unsigned char*>(workspace);
  bf16* kimg = reinterpret_cast<bf16*>(w);
  bf16* qimg = reinterpret_cast<bf16*>(w + align256(ody_attn_images_bytes(p.B, p.Lk, p.Hkv)));
  bf16* doimg = reinterpret_cast<bf16*>(w + align256(ody_attn_images_bytes(p.B, p.Lk, p.Hkv)) +
                                        align256(ody_attn_images_bytes(p.B, p.Lq, p.Hq)));
  bf16* stats = reinterpret_cast<bf16*>(reinterpret_cast<unsigned char*>(doimg) +
                                        align256(ody_attn_images_bytes(p.B, p.Lq, p.Hq)));
  int rc;
  // everything that depends on q, dout, out and lse only: delta, Q / dO images, start values
  if (!p.reuse_query_side && (rc = ody_launch_attn_bwd_prepass(p, qimg, doimg, stats, st))) return rc;
  if ((rc = ody_launch_attn_images(p.k, p.sk, p.B, p.Lk, p.Hkv, kimg, nullptr, 0, st))) return rc;
  const int key_blocks = (p.Lk + KV_BN - 1) / KV_BN;
  float* part = reinterpret_cast<float*>(
      reinterpret_cast<unsigned char*>(stats) +
      align256((size_t)p.B * p.Hq * ((p.Lq + KV_BQ - 1) / KV_BQ) * KV_STAT_ELEMS * sizeof(bf16)));
  const int qparts = query_parts(p.B, p.Lq, p.Lk, p.Hq, p.Hkv, p.causal != 0);
  if (p.group == 1 && qparts == 1) {
    if (p.ds)
      ODY_LAUNCH("attn_bwd_dkdv_pipe", st, (attn_bwd_dkdv_pipe_kernel<false, true>), dim3(key_blocks * p.Hkv * p.B),
                 dim3(KV_THREADS), smem_kv, p, qimg, doimg, stats, nullptr, 1);
    else
      ODY_LAUNCH("attn_bwd_dkdv_pipe", st, (attn_bwd_dkdv_pipe_kernel<false, false>), dim3(key_blocks * p.Hkv * p.B),
                 dim3(KV_THREADS), smem_kv, p, qimg, doimg, stats, nullptr, 1);
    if ((rc = ody_check_launch("attn_bwd_dkdv_pipe"))) return rc;
  } else {
    if (p.ds)
      ODY_LAUNCH("attn_bwd_dkdv_pipe", st, (attn_bwd_dkdv_pipe_kernel<true, true>), dim3(key_blocks * p.Hq * qparts * p.B),
                 dim3(KV_THREADS), smem_kv, p, qimg, doimg, stats, part, qparts);
    else
      ODY_LAUNCH("attn_bwd_dkdv_pipe", st, (attn_bwd_dkdv_pipe_kernel<true, false>), dim3(key_blocks * p.Hq * qparts * p.B),
                 dim3(KV_THREADS), smem_kv, p, qimg, doimg, stats, part, qparts);
    if ((rc = ody_check_launch("attn_bwd_dkdv_pipe"))) return rc;
    const int64_t n8 = (int64_t)p.B * p.Hkv * p.Lk * (D / 8);
    ODY_LAUNCH("attn_bwd_group_sum", st, attn_bwd_group_sum_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, p,
               part, qparts);
    if ((rc = ody_check_launch("attn_bwd_group_sum"))) return rc;
  }
  dim3 gq(((p.Lq + DQ_BM - 1) / DQ_BM) * p.Hq * p.B);
  if (p.ds) {
    // what ody_attn_bwd_pipe_ds_bytes promised: whole 256-row blocks on both sides, queries and keys aligned
    ODY_REQUIRE(p.Lq % KV_BN == 0 && p.Lk % KV_BN == 0 && (!p.causal || p.off == 0) && KV_BN == DQ_BM, ODY_ERR_UNSUPPORTED,
                "attn_bwd: kept dS needs multiples of %d rows on both sides and, if causal, as many keys as queries", KV_BN);
    const int kparts = key_parts(p.B, p.Lq, p.Lk, p.Hq, p.causal != 0);
    ODY_LAUNCH("attn_bwd_dq_kept", st, attn_bwd_dq_kept_kernel, dim3(gq.x * kparts), dim3(DQ_THREADS), smem_qs, p, kimg, kparts,
               part);
    if ((rc = ody_check_launch("attn_bwd_dq_kept")) || kparts == 1) return rc;
    const int64_t n8 = (int64_t)p.B * p.Lq * p.Hq * (D / 8);
    ODY_LAUNCH("attn_bwd_dq_sum", st, attn_bwd_dq_sum_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, p, part, kparts);
    return ody_check_launch("attn_bwd_dq_sum");
  }
  const int kparts = key_parts(p.B, p.Lq, p.Lk, p.Hq, p.causal != 0);
  ODY_LAUNCH("attn_bwd_dq_pipe", st, attn_bwd_dq_pipe_kernel, dim3(gq.x * kparts), dim3(DQ_THREADS), smem_q, p, kimg, kparts,
             part);
  if ((rc = ody_check_launch("attn_bwd_dq_pipe")) || kparts == 1) return rc;
  const int64_t n8 = (int64_t)p.B * p.Lq * p.Hq * (D / 8);
  ODY_LAUNCH("attn_bwd_dq_sum", st, attn_bwd_dq_sum_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, p, part, kparts);
  return ody_check_launch("attn_bwd_dq_sum");
}
