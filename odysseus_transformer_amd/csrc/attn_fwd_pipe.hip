// Flash-attention forward, head_dim 128, bf16: software-pipelined kernel.
//
// Dataflow per wavefront (lane = 32*g + i owns query column i of each of its 2 query
// tiles, so every per-query quantity is a per-lane scalar):
//
//   S^T (keys x queries) = K . Q^T          A: K rows from LDS, B: Q^T in registers
//   O^T (d x queries)   += V^T . P^T        A: V^T rows from LDS (transposed image written
//                                              by a pre-pass), B: P^T = the S^T accumulators
//
// A step covers 32 keys x 64 queries per wavefront (256 queries per workgroup): every
// operand fragment read from LDS feeds two MFMAs and every K / V tile fetched from L2
// serves 256 queries.  The step overlaps the matrix pipe with the vector ALUs:
//
//   step j :  S(j+1) = K(j+1) Q^T      (MFMA)   ||   P(j) = exp2(S(j) c - ref)   (VALU)
//             O     += V(j) P(j)       (MFMA)   ||   row max of S(j+1)           (VALU)
//
// written as 32 fenced slots {prefetch an operand for a later MFMA, one MFMA, a slice of
// vector work}.  K runs ahead of V: the K ring holds three 64-key tiles, the V ring two
// images, both filled by direct global->LDS loads (no staging registers, no LDS stores).
//
// The softmax reference of a query is FIXED by its first 32 keys; exp2 of later scores
// uses it as long as they exceed it by less than 2^64 (fp32 sums and bf16 P have the
// exponent range for that), which holds for any sane input.  Nothing in this kernel
// rescales O.  A workgroup that meets a score beyond the window sets its flag in the
// workspace, and the launcher's follow-up kernel (the online-rescaling kernel of
// attn_fwd_mfma.hip, which exits at once for unflagged blocks) recomputes its block.
// Any reference gives the same out = O / l and lse = ref + log(l).
#include <type_traits>
#include "attn_params.h"
#include "attn_tile.h"

namespace {

using namespace tile128;

constexpr int D = 128, KS = D / 16, DT = D / 32, BN = 64, QT = 2, WQ = 32 * QT, BM = 4 * WQ;
constexpr float LAZY_LOG2 = 64.0f;

// nothing may be moved across a fence by the instruction scheduler
#define FENCE() __builtin_amdgcn_sched_barrier(0)


struct SoftState {
  float ref_c;   // reference * scale*log2e (0 while no key has been seen)
  float thr;     // raw score above which the reference must move (-inf while no key has been seen)
  float l[4];    // this lane's partial row sums (independent chains)
};

__global__ __launch_bounds__(256) void attn_fwd_pipe_kernel(const AttnParams p, const bf16* __restrict__ vimg,
                                                            int* __restrict__ bail_flags) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* Kring = reinterpret_cast<bf16*>(smem_raw);   // [3][TILE_ELEMS]
  bf16* Vring = Kring + 3 * TILE_ELEMS;              // [2][IMG_ELEMS]

  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g = lane >> 5, i = lane & 31;
  const BlockCoord bc = ody_block_coord(p.Hq, p.B);
  const int nqb = gridDim.x / (p.Hq * p.B);
  const int qblk = p.causal ? (nqb - 1 - bc.rank) : bc.rank;   // heaviest blocks first
  const int h = bc.h, b = bc.b, hk = h / p.group;
  const int q0 = qblk * BM, wq0 = q0 + wave * WQ;

  const bf16* qp = static_cast<const bf16*>(p.q) + b * p.sq.b + h * p.sq.h;
  const bf16* kp = static_cast<const bf16*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const int kv_tiles = (p.Lk + BN - 1) / BN;
  const bf16* vp = vimg + ((int64_t)b * p.Hkv + hk) * kv_tiles * IMG_ELEMS;

  const int q_hi = min(q0 + BM, p.Lq) - 1;
  int n_end = p.causal ? min(p.Lk, q_hi + p.off + 1) : p.Lk;
  if (n_end < 0) n_end = 0;
  const int ntiles = (n_end + BN - 1) / BN;
  const int nsub = 2 * ntiles;                       // 32-key sub-tiles
  // sub-tiles [0, sub_full) need no mask for any wavefront of the block
  int n_full = p.Lk / BN;
  if (p.causal) n_full = min(n_full, max(0, (q0 + p.off + 1) / BN));
  const int sub_full = 2 * min(n_full, ntiles);

  if (ntiles > 0) {
    load_tile_async(Kring, kp, p.sk.l, 0, p.Lk, wave, lane);
    load_image_async(Vring, vp, wave, lane);
    if (ntiles > 1) load_tile_async(Kring + TILE_ELEMS, kp, p.sk.l, BN, p.Lk, wave, lane);
  }

  bf16x8 qf[QT][KS];
  int lim[QT];
#pragma unroll
  for (int qt = 0; qt < QT; qt++) {
    const int qi = wq0 + 32 * qt + i;
    lim[qt] = p.causal ? min(p.Lk - 1, qi + p.off) : p.Lk - 1;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (qi < p.Lq) qf[qt][ks] = *reinterpret_cast<const bf16x8*>(qp + (int64_t)qi * p.sq.l + 16 * ks + 8 * g);
      else qf[qt][ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }

  f32x16 o[QT][DT];
#pragma unroll
  for (int qt = 0; qt < QT; qt++)
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[qt][dt][r] = 0.f;
  SoftState st[QT];
#pragma unroll
  for (int qt = 0; qt < QT; qt++) st[qt] = SoftState{0.f, -INFINITY, {0.f, 0.f, 0.f, 0.f}};
  const float c2 = p.scale_log2e;
  const float lazy_raw = LAZY_LOG2 / c2;
  const int rbase = row_frag_base(g, i), ibase = image_frag_base(g, i);

  f32x16 sA[QT], sB[QT];

  // per-thread element offsets of the 4 direct loads of a K tile (row 4*grp + (lane >> 4), chunk lane & 15)
  unsigned koff[4];
#pragma unroll
  for (int j = 0; j < 4; j++) koff[j] = (unsigned)((4 * (4 * j + wave) + (lane >> 4)) * p.sk.l + 8 * (lane & 15));
  // a K tile whose 64 rows all exist: uniform base + per-lane offset; the ragged last tile clamps rows
  auto load_k = [&](bf16* lds_tile, int row0) {
    if (row0 + ROWS <= p.Lk) {
      const bf16* tb = kp + (int64_t)row0 * p.sk.l;
#pragma unroll
      for (int j = 0; j < 4; j++)
        __builtin_amdgcn_global_load_lds((global_void_ptr)(tb + koff[j]),
                                         (lds_void_ptr)(lds_tile + (4 * j + wave) * GROUP_ELEMS), 16, 0, 0);
    } else {
      load_tile_async(lds_tile, kp, p.sk.l, row0, p.Lk, wave, lane);
    }
  };

  // ---- building blocks -------------------------------------------------------------
  auto mask1 = [&](f32x16 (&s)[QT], int key0, int kt, int e) {
    const int qt = e >> 4, r = e & 15;
    if (key0 + acc_tile_row(r, g, kt) > lim[qt]) s[qt][r] = -INFINITY;
  };
  // The reference is fixed by the first sub-tile (key 0 is in it, and every query that sees
  // any key sees key 0).  A later score beyond the lazy window only raises `bail`.
  bool bail = false;
  auto set_reference = [&](const float (&mx)[QT]) {
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
      const bool seen = mx[qt] != -INFINITY;
      st[qt].ref_c = seen ? mx[qt] * c2 : 0.f;
      st[qt].thr = seen ? mx[qt] + lazy_raw : INFINITY;
    }
  };
  auto check_window = [&](const float (&mx)[QT]) {
    bool any = false;
#pragma unroll
    for (int qt = 0; qt < QT; qt++) any = any || (mx[qt] > st[qt].thr);
    bail = bail || (__builtin_amdgcn_ballot_w64(any) != 0);
  };
  // P element e (0..31: query tile e>>4, register e&15) of the current sub-tile: exp2, row sum, bf16 pack
  auto prob1 = [&](const f32x16 (&s)[QT], bf16x8 (&pb)[QT][2], int e) {
    const int qt = e >> 4, r = e & 15;
    const float x = ody_exp2(fmaf(s[qt][r], c2, -st[qt].ref_c));
    st[qt].l[r & 3] += x;
    pb[qt][r >> 3][r & 7] = (bf16)x;
  };
  // top of a KV tile: own loads landed, every wavefront done with the previous tile
  auto sync_and_prefetch = [&](int t) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (t + 2 < ntiles) load_k(Kring + ((t + 2) % 3) * TILE_ELEMS, (t + 2) * BN);
    if (t + 1 < ntiles)
      load_image_async(Vring + ((t + 1) & 1) * IMG_ELEMS, vp + (int64_t)(t + 1) * IMG_ELEMS, wave, lane);
  };
  // S of sub-tile j (32 keys x 64 queries), unpipelined: prologue only
  auto qk_plain = [&](int j, f32x16 (&s)[QT]) {
    const bf16* Kt = Kring + ((j >> 1) % 3) * TILE_ELEMS;
#pragma unroll
    for (int qt = 0; qt < QT; qt++)
#pragma unroll
      for (int r = 0; r < 16; r++) s[qt][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const bf16x8 a = row_frag(Kt, rbase, ks, j & 1);
#pragma unroll
      for (int qt = 0; qt < QT; qt++) s[qt] = mfma32(a, qf[qt][ks], s[qt]);
    }
  };
  // row maxima of a complete S tile (after masking), both halves of the wavefront combined
  auto rowmax = [&](const f32x16 (&s)[QT], float (&mx)[QT]) {
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
      float m = s[qt][0];
#pragma unroll
      for (int r = 1; r < 16; r++) m = fmaxf(m, s[qt][r]);
      mx[qt] = half_swap_max(m);
    }
  };
  // The pipelined step for sub-tile j (plain sub-tiles only): consumes s_cur = S(j), produces
  // s_nxt = S(j+1) and its row maxima.
  //   slots  0..15: S(j+1) += K Q^T   with   P(j) elements 0..23
  //   slots 16..31: O += V(j) P(j)    with   P(j) elements 24..31, row max of S(j+1)
  auto step = [&](int j, f32x16 (&s_cur)[QT], f32x16 (&s_nxt)[QT], float (&mx)[QT]) {
    if ((j & 1) == 0) sync_and_prefetch(j >> 1);
    const int kt = j & 1, ktn = (j + 1) & 1;
    const bf16* Kt = Kring + (((j + 1) >> 1) % 3) * TILE_ELEMS;
    const bf16* Vt = Vring + ((j >> 1) & 1) * IMG_ELEMS;
    bf16x8 pb[QT][2];
    constexpr int KPF = 4, VPF = 4;
    bf16x8 kfr[KPF];
#pragma unroll
    for (int n = 0; n < KPF; n++) kfr[n] = row_frag(Kt, rbase, n, ktn);
    FENCE();
#pragma unroll
    for (int n = 0; n < 16; n++) {
      const int ks = n >> 1, qt = n & 1;
      if (ks == 0) s_nxt[qt] = mfma32(kfr[ks % KPF], qf[qt][ks], f32x16{0});
      else s_nxt[qt] = mfma32(kfr[ks % KPF], qf[qt][ks], s_nxt[qt]);
      if (qt == 1 && ks + KPF < KS) kfr[ks % KPF] = row_frag(Kt, rbase, ks + KPF, ktn);
#pragma unroll
      for (int e = (3 * n) >> 1; e < (3 * (n + 1)) >> 1; e++) prob1(s_cur, pb, e);
      FENCE();
    }
    bf16x8 vfr[VPF];
#pragma unroll
    for (int qt = 0; qt < QT; qt++) mx[qt] = -INFINITY;
    // PV slot n: fragment f = n >> 1 (ss = f >> 2, dt = f & 3), query tile n & 1
#pragma unroll
    for (int f = 0; f < VPF; f++) vfr[f] = image_frag(Vt, ibase, f & 3, f >> 2, kt);
    FENCE();
#pragma unroll
    for (int n = 0; n < 16; n++) {
      const int f = n >> 1, qt = n & 1, dt = f & 3, ss = f >> 2;
      if (n < 8) prob1(s_cur, pb, 24 + n);
      o[qt][dt] = mfma32(vfr[f % VPF], pb[qt][ss], o[qt][dt]);
      if (qt == 1 && f + VPF < 8) vfr[f % VPF] = image_frag(Vt, ibase, (f + VPF) & 3, (f + VPF) >> 2, kt);
#pragma unroll
      for (int e = 2 * n; e < 2 * n + 2; e++) mx[e >> 4] = fmaxf(mx[e >> 4], s_nxt[e >> 4][e & 15]);
      FENCE();
    }
#pragma unroll
    for (int qt = 0; qt < QT; qt++) mx[qt] = half_swap_max(mx[qt]);
    check_window(mx);
  };
  // The plain (unpipelined) treatment of sub-tile j whose S and row maxima are at hand: moves
  // the reference if needed, then P and O += V P.  Used where the pipeline does not reach:
  // the first sub-tile, the masked ones near the diagonal, the last one, and whenever the
  // lazy reference has to move.
  auto finish = [&](int j, f32x16 (&s)[QT]) {
    if ((j & 1) == 0) sync_and_prefetch(j >> 1);
    const bf16* Vt = Vring + ((j >> 1) & 1) * IMG_ELEMS;
    bf16x8 pb[QT][2];
#pragma unroll
    for (int e = 0; e < 32; e++) prob1(s, pb, e);
#pragma unroll
    for (int f = 0; f < 8; f++) {
      const bf16x8 a = image_frag(Vt, ibase, f & 3, f >> 2, j & 1);
#pragma unroll
      for (int qt = 0; qt < QT; qt++) o[qt][f & 3] = mfma32(a, pb[qt][f >> 2], o[qt][f & 3]);
    }
  };
  // S(j) and its row maxima, computed on the spot
  auto prepare = [&](int j, f32x16 (&s)[QT], float (&mx)[QT]) {
    qk_plain(j, s);
    if (j >= sub_full) {
#pragma unroll
      for (int e = 0; e < 32; e++) mask1(s, (j >> 1) * BN, j & 1, e);
    }
    rowmax(s, mx);
    if (j == 0) set_reference(mx); else check_window(mx);
  };

  // ---- main loop ----------------------------------------------------------------------
  if (nsub > 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    float mx[QT];
    prepare(0, sA, mx);
    int j = 0;
    while (true) {
      finish(j, sA);
      if (++j == nsub) break;
      prepare(j, sA, mx);
      // pipelined run over plain sub-tiles (S(j+1) needs no mask); leaves S(j) in sA
      while (j + 2 < sub_full) {
        step(j, sA, sB, mx);
        step(j + 1, sB, sA, mx);
        j += 2;
      }
    }
  }

  // ---- epilogue ----------------------------------------------------------------------
  if (bail && lane == 0) atomicOr(bail_flags + ((int64_t)b * p.Hq + h) * nqb + qblk, 1);
  bf16* op = static_cast<bf16*>(p.out) + b * p.so.b + h * p.so.h;
  float* lsep = p.lse + ((int64_t)b * p.Hq + h) * p.Lq;
#pragma unroll
  for (int qt = 0; qt < QT; qt++) {
    const int qi = wq0 + 32 * qt + i;
    const float lt = half_swap_sum((st[qt].l[0] + st[qt].l[1]) + (st[qt].l[2] + st[qt].l[3]));
    const float inv = lt > 0.f ? 1.f / lt : 0.f;
    if (qi < p.Lq) {
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int a = 0; a < 4; a++) {
          bf16x4 w;
#pragma unroll
          for (int e = 0; e < 4; e++) w[e] = (bf16)(o[qt][dt][4 * a + e] * inv);
          *reinterpret_cast<bf16x4*>(op + (int64_t)qi * p.so.l + 32 * dt + 8 * a + 4 * g) = w;
        }
      if (g == 0) lsep[qi] = lt > 0.f ? (st[qt].ref_c + __log2f(lt)) * ODY_LN2 : -INFINITY;
    }
  }
}

}  // namespace

size_t ody_attn_fwd_pipe_workspace(int B, int Lq, int Lk, int Hq, int Hkv) {
  const size_t flags = ((size_t)B * Hq * ((Lq + BM - 1) / BM) * sizeof(int) + 255) & ~(size_t)255;
  return flags + ody_attn_images_bytes(B, Lk, Hkv);
}

// workspace: [bail flags | transposed images of V]
int ody_launch_attn_fwd_pipe(const AttnParams& p, void* workspace, hipStream_t st) {
  constexpr size_t smem = (size_t)3 * TILE_BYTES + 2 * IMG_BYTES;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_fwd_pipe_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      ody_set_error("attn_fwd: hipFuncSetAttribute failed: %s", hipGetErrorString(e));
      return ODY_ERR_LAUNCH;
    }
    attr_set = true;
  }
  const int nqb = (p.Lq + BM - 1) / BM;
  const int nflags = p.B * p.Hq * nqb;
  int* flags = static_cast<int*>(workspace);
  bf16* images = reinterpret_cast<bf16*>(static_cast<char*>(workspace) + (((size_t)nflags * sizeof(int) + 255) & ~(size_t)255));
  int rc = ody_launch_attn_images(p.v, p.sv, p.B, p.Lk, p.Hkv, images, flags, nflags, st);
  if (rc) return rc;
  dim3 grid(nqb * p.Hq * p.B);
  ODY_LAUNCH("attn_fwd_pipe", st, attn_fwd_pipe_kernel, grid, dim3(256), smem, p, images, flags);
  rc = ody_check_launch("attn_fwd_pipe");
  if (rc) return rc;
  return ody_launch_attn_fwd_mfma_flagged(p, flags, BM, st);
}

