// Flash-attention forward, head_dim 128, bf16, on the tile machinery of attn_tile.h with two
// wavefronts per SIMD: 8 wavefronts x 32 queries per block, so that one wavefront's vector work
// (exp2, row sums, bf16 packing) runs under the other's MFMAs.  Query-stationary, computed
// transposed, lane = query column:
//
//      S^T = K Q^T            A: K rows (LDS tile)          B: Q^T (registers)
//      P^T = exp2(S^T c - m)  per-lane reference m, per-lane row sum
//      O^T += V^T P^T         A: V^T (transposed image)     B: P^T = accumulator layout of S^T
//
// The reference m of a query is fixed by its first 32 keys (key 0 is among them, and a query that
// sees any key sees key 0): the loop neither tracks maxima nor rescales O.  A later score that
// outgrows the reference by more than fp32 can hold shows up as a row sum that overflowed; the
// 256-query block is then flagged and redone by the online-rescaling kernel.
//
// A call with few query blocks (16384 queries are 64 per head; the off-diagonal steps of a zigzag ring have 32) leaves
// compute units idle or, under a causal mask, waiting for the one with the longest block: then every block's key range
// is cut into 2 or 4 parts, one block per (query block, part); each writes its normalised partial result and
// log-sum-exp in fp32 and a small kernel merges the parts with the arithmetic of the ring's block merge.
#include "attn_params.h"
#include "attn_tile.h"

namespace {

using namespace tile128;

constexpr int D = 128, KS = D / 16, DT = D / 32, BN = 64;
constexpr int FW_WAVES = 8, FW_BM = 32 * FW_WAVES, FW_THREADS = 64 * FW_WAVES;
constexpr int FW_STAGE = TILE_ELEMS + IMG_ELEMS;   // K tile, V^T image
static_assert(FW_WAVES == 8, "the load split and the vmcnt waits assume 8 wavefronts");
#define FENCE() __builtin_amdgcn_sched_barrier(0)

// nsplit > 1: block id = split + nsplit * (the usual id), the block takes part `split` of its tiles; part_out
// [split][B][Lq][Hq][D] and part_lse [split][B][Hq][Lq] in fp32 take the place of p.out / p.lse.  Under a causal mask a
// later part may start beyond the first keys of some of its queries: their reference is then 0 instead of a score,
// which the overflow flag covers like any other reference that turns out too low.
__global__ __launch_bounds__(FW_THREADS) void attn_fwd_w8_kernel(const AttnParams p, const bf16* __restrict__ vimg,
                                                                  int* __restrict__ bail_flags, int nsplit,
                                                                  float* __restrict__ part_out,
                                                                  float* __restrict__ part_lse) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* ring = reinterpret_cast<bf16*>(smem_raw);   // [3][FW_STAGE]

  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g = lane >> 5,
            i = lane & 31;
  simd_stagger(tid);
  const int split = blockIdx.x % nsplit;
  const BlockCoord bc = ody_block_coord_of(blockIdx.x / nsplit, p.Hq, p.B);
  const int nqb = gridDim.x / (p.Hq * p.B * nsplit);
  const int qblk = p.causal ? (nqb - 1 - bc.rank) : bc.rank;   // heaviest blocks first
  const int h = bc.h, b = bc.b, hk = h / p.group;
  const int q0 = qblk * FW_BM, wq0 = q0 + wave * 32, qi = wq0 + i;

  const bf16* qp = static_cast<const bf16*>(p.q) + b * p.sq.b + h * p.sq.h;
  const bf16* kp = static_cast<const bf16*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const int kv_tiles = (p.Lk + BN - 1) / BN;
  const bf16* vp = vimg + ((int64_t)b * p.Hkv + hk) * kv_tiles * IMG_ELEMS;

  const int q_hi = min(q0 + FW_BM, p.Lq) - 1;
  int n_end = p.causal ? min(p.Lk, q_hi + p.off + 1) : p.Lk;
  if (n_end < 0) n_end = 0;
  int ntiles = (n_end + BN - 1) / BN;
  int n_full = p.Lk / BN;   // tiles [0, n_full) need no mask for any wavefront of the block
  if (p.causal) n_full = min(n_full, max(0, (q0 + p.off + 1) / BN));
  n_full = min(n_full, ntiles);
  // this block's part of the tiles: [t_first, ntiles)
  int t_first = 0;
  if (nsplit > 1) {
    const int per = (ntiles + nsplit - 1) / nsplit;
    t_first = min(split * per, ntiles);
    ntiles = min(t_first + per, ntiles);
  }

  // half j (0/1) of the direct loads of stage t: 2 loads per wavefront
  auto load_part = [&](bf16* st, int t, int j) {
    const int grp = FW_WAVES * j + wave;
    int row = t * BN + 4 * grp + (lane >> 4);
    row = row < p.Lk ? row : p.Lk - 1;
    __builtin_amdgcn_global_load_lds((global_void_ptr)(kp + (int64_t)row * p.sk.l + 8 * (lane & 15)),
                                     (lds_void_ptr)(st + grp * GROUP_ELEMS), 16, 0, 0);
    __builtin_amdgcn_global_load_lds((global_void_ptr)(vp + (int64_t)t * IMG_ELEMS + (grp * 64 + lane) * 8),
                                     (lds_void_ptr)(st + TILE_ELEMS + grp * 512), 16, 0, 0);
  };
  for (int t = t_first; t < t_first + 2 && t < ntiles; t++) {
    load_part(ring + ((t - t_first) % 3) * FW_STAGE, t, 0);
    load_part(ring + ((t - t_first) % 3) * FW_STAGE, t, 1);
  }

  bf16x8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    if (qi < p.Lq) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + (int64_t)qi * p.sq.l + 16 * ks + 8 * g);
    else qf[ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
  }
  // Q^T must have ARRIVED before the loop: left pending, the compiler places its wait for these register loads at
  // their first use, inside the loop, as a wait for every load in flight -- and the ring's direct loads, which are
  // issued two turns ahead, would have to land within one.
#pragma unroll
  for (int ks = 0; ks < KS; ks++) asm volatile("" : "+v"(qf[ks]));
  const int lim = p.causal ? min(p.Lk - 1, qi + p.off) : p.Lk - 1;   // last key this lane's query sees
  const float c2 = p.scale_log2e;
  const int rbase = row_frag_base(g, i), ibase = image_frag_base(g, i);

  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[dt][r] = 0.f;
  float ref_c = 0.f;                        // reference * scale * log2(e); 0 for a query that sees no key
  float l4[4] = {0.f, 0.f, 0.f, 0.f};       // this lane's partial row sums (independent chains)

  // One 64-key tile against this wavefront's 32 queries, as two 32-key sub-tiles kt = 0, 1 whose
  // S^T accumulate in two independent MFMA chains: 16 MFMAs for S^T, the vector work, 16 MFMAs for O^T.
  auto tile = [&](const bf16* st, int t, bool masked, bool first) {
    const bf16* Kt = st;
    const bf16* Vi = st + TILE_ELEMS;
    constexpr int PF = 2;   // k-steps of K fragments in flight (two fragments each)
    bf16x8 kfr[PF][2];
#pragma unroll
    for (int n = 0; n < PF; n++)
#pragma unroll
      for (int kt = 0; kt < 2; kt++) kfr[n][kt] = row_frag(Kt, rbase, n, kt);
    f32x16 s[2];
    FENCE();
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
        if (ks == 0) s[kt] = mfma32(kfr[0][kt], qf[0], f32x16{0});
        else s[kt] = mfma32(kfr[ks % PF][kt], qf[ks], s[kt]);
      }
      if (ks + PF < KS) {
#pragma unroll
        for (int kt = 0; kt < 2; kt++) kfr[ks % PF][kt] = row_frag(Kt, rbase, ks + PF, kt);
      }
      FENCE();
    }
    constexpr int VPF = 4;
    bf16x8 vfr[VPF];
#pragma unroll
    for (int n = 0; n < VPF; n++) vfr[n] = image_frag(Vi, ibase, n & 3, 0, 0);
    if (masked) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          if (t * BN + acc_tile_row(r, g, kt) > lim) s[kt][r] = -INFINITY;
    }
    if (first) {   // the reference: the largest score among the 32 keys of sub-tile 0 (key 0 is one of them)
      float m = s[0][0];
#pragma unroll
      for (int r = 1; r < 16; r++) m = fmaxf(m, s[0][r]);
      m = half_swap_max(m);
      ref_c = (m != -INFINITY) ? m * c2 : 0.f;
    }
    bf16x8 pb[2][2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float x = ody_exp2(fmaf(s[kt][r], c2, -ref_c));
        l4[r & 3] += x;
        pb[kt][r >> 3][r & 7] = (bf16)x;
      }
    FENCE();
    // PV step n: k-step (kt, ss) = (n >> 3, (n >> 2) & 1), output tile dt = n & 3
#pragma unroll
    for (int n = 0; n < 16; n++) {
      const int dt = n & 3, ss = (n >> 2) & 1, kt = n >> 3;
      o[dt] = mfma32(vfr[n % VPF], pb[kt][ss], o[dt]);
      if (n + VPF < 16) {
        const int m = n + VPF;
        vfr[n % VPF] = image_frag(Vi, ibase, m & 3, (m >> 2) & 1, m >> 3);
      }
      FENCE();
    }
  };

  for (int t = t_first; t < ntiles; t++) {
    // stage t landed (the 4 loads of stage t+1 may still be in flight), everyone done with stage t-1
    if (t + 1 < ntiles) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (t + 2 < ntiles) {
      load_part(ring + ((t + 2 - t_first) % 3) * FW_STAGE, t + 2, 0);
      load_part(ring + ((t + 2 - t_first) % 3) * FW_STAGE, t + 2, 1);
    }
    // every key of the tile is after this wavefront's queries (never the case for tile 0)
    const bool dead = p.causal && t * BN > wq0 + 31 + p.off;
    if (!dead) tile(ring + ((t - t_first) % 3) * FW_STAGE, t, t >= n_full, t == t_first);
  }

  // ---- epilogue
  const float lt = half_swap_sum((l4[0] + l4[1]) + (l4[2] + l4[3]));
  if (__builtin_amdgcn_ballot_w64(!(lt < 0x1p100f)) != 0 && lane == 0)
    atomicOr(bail_flags + ((int64_t)b * p.Hq + h) * nqb + qblk, 1);
  if (nsplit > 1) {
    if (qi < p.Lq) {   // this part's normalised result and log-sum-exp, for the merge kernel
      float* op = part_out + ((((int64_t)split * p.B + b) * p.Lq + qi) * p.Hq + h) * D;
      const float inv = lt > 0.f ? 1.f / lt : 0.f;
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int a = 0; a < 4; a++) {
          f32x4 w;
#pragma unroll
          for (int e = 0; e < 4; e++) w[e] = o[dt][4 * a + e] * inv;
          *reinterpret_cast<f32x4*>(op + 32 * dt + 8 * a + 4 * g) = w;
        }
      if (g == 0)
        part_lse[(((int64_t)split * p.B + b) * p.Hq + h) * p.Lq + qi] = lt > 0.f ? (ref_c + __log2f(lt)) * ODY_LN2 : -INFINITY;
    }
    return;
  }
  if (qi < p.Lq) {
    bf16* op = static_cast<bf16*>(p.out) + b * p.so.b + h * p.so.h + (int64_t)qi * p.so.l;
    const float inv = lt > 0.f ? 1.f / lt : 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int a = 0; a < 4; a++) {
        bf16x4 w;
#pragma unroll
        for (int e = 0; e < 4; e++) w[e] = (bf16)(o[dt][4 * a + e] * inv);
        *reinterpret_cast<bf16x4*>(op + 32 * dt + 8 * a + 4 * g) = w;
      }
    if (g == 0) p.lse[((int64_t)b * p.Hq + h) * p.Lq + qi] = lt > 0.f ? (ref_c + __log2f(lt)) * ODY_LN2 : -INFINITY;
  }
}

// out, lse of a query from its `nsplit` parts: lse = log sum_s exp(lse_s), out = sum_s exp(lse_s - lse) out_s -- the
// ring merge (decoder/ring.py:30-37 of the reference reaches it through ring_flash_attn) over all parts at once.
// One thread per 4 elements of a (query, head) row.
__global__ __launch_bounds__(256) void attn_fwd_split_merge_kernel(const AttnParams p, int nsplit,
                                                                   const float* __restrict__ part_out,
                                                                   const float* __restrict__ part_lse) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;   // over B * Lq * Hq * D / 4
  const int64_t total = (int64_t)p.B * p.Lq * p.Hq * (D / 4);
  if (idx >= total) return;
  const int d4 = idx % (D / 4);
  const int h = (idx / (D / 4)) % p.Hq;
  const int qi = (idx / ((int64_t)(D / 4) * p.Hq)) % p.Lq;
  const int b = idx / ((int64_t)(D / 4) * p.Hq * p.Lq);
  const int64_t plane_o = (int64_t)p.B * p.Lq * p.Hq * D, plane_l = (int64_t)p.B * p.Hq * p.Lq;
  const int64_t li = ((int64_t)b * p.Hq + h) * p.Lq + qi;
  float m = -INFINITY;
  for (int s = 0; s < nsplit; s++) m = fmaxf(m, part_lse[s * plane_l + li]);
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float wsum = 0.f;
  if (m != -INFINITY) {
    const float* po = part_out + (((int64_t)b * p.Lq + qi) * p.Hq + h) * D + 4 * d4;
    for (int s = 0; s < nsplit; s++) {
      const float w = __expf(part_lse[s * plane_l + li] - m);   // exp(-inf) = 0 for a part that saw no key
      wsum += w;
      acc += w * *reinterpret_cast<const f32x4*>(po + s * plane_o);
    }
  }
  const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
  bf16x4 w;
#pragma unroll
  for (int e = 0; e < 4; e++) w[e] = (bf16)(acc[e] * inv);
  *reinterpret_cast<bf16x4*>(static_cast<bf16*>(p.out) + b * p.so.b + h * p.so.h + (int64_t)qi * p.so.l + 4 * d4) = w;
  if (d4 == 0) p.lse[li] = wsum > 0.f ? m + __logf(wsum) : -INFINITY;
}

inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

// Parts of a query block's key range.  With fewer blocks than it takes to keep the chip's 256 compute units busy and
// balanced -- one block each when all blocks are equally long (fully visible keys), two each when they are not (under
// a causal mask block i is i + 1 tiles long, and only with a second, lighter block per unit does the heaviest-first
// order even that out) -- the range is cut into 2 or 4 parts of at least 8 tiles (on average, when causal).
int key_splits(int B, int Lq, int Lk, int Hq, bool causal) {
  const int64_t blocks = (int64_t)B * Hq * ((Lq + FW_BM - 1) / FW_BM);
  const int64_t want = causal ? 512 : 256;
  const int tiles = ((causal ? min(Lk, Lq + max(Lk - Lq, 0)) : Lk) + BN - 1) / BN;
  int s = 1;
  while (s < 4 && blocks * s * 2 <= want && tiles >= 16 * s) s *= 2;
  return s;
}

}  // namespace

// workspace: [flags of the 256-query blocks | transposed images of V | fp32 parts of a key-split call: out, lse]
size_t ody_attn_fwd_w8_workspace(int B, int Lq, int Lk, int Hq, int Hkv, bool with_split) {
  const size_t flags = align256((size_t)B * Hq * ((Lq + FW_BM - 1) / FW_BM) * sizeof(int));
  size_t n = flags + align256(ody_attn_images_bytes(B, Lk, Hkv));
  const int ns = with_split ? max(key_splits(B, Lq, Lk, Hq, false), key_splits(B, Lq, Lk, Hq, true)) : 1;
  if (ns > 1) n += align256((size_t)ns * B * Lq * Hq * D * sizeof(float)) + align256((size_t)ns * B * Hq * Lq * sizeof(float));
  return n;
}

int ody_launch_attn_fwd_w8(const AttnParams& p, void* workspace, size_t workspace_bytes, hipStream_t st) {
  constexpr size_t smem = (size_t)3 * FW_STAGE * sizeof(bf16);
  int rc = ody_allow_dynamic_lds(reinterpret_cast<const void*>(&attn_fwd_w8_kernel), smem, "attn_fwd");
  if (rc) return rc;
  const int nqb = (p.Lq + FW_BM - 1) / FW_BM;
  const int nflags = p.B * p.Hq * nqb;
  char* w = static_cast<char*>(workspace);
  int* flags = reinterpret_cast<int*>(w);
  bf16* images = reinterpret_cast<bf16*>(w + align256((size_t)nflags * sizeof(int)));
  rc = ody_launch_attn_images(p.v, p.sv, p.B, p.Lk, p.Hkv, images, flags, nflags, st);
  if (rc) return rc;
  // the key split, where the caller's workspace has room for the parts (the allocation-free entry point's fixed
  // scratch may not)
  int ns = key_splits(p.B, p.Lq, p.Lk, p.Hq, p.causal != 0);
  if (ns > 1 && workspace_bytes < ody_attn_fwd_w8_workspace(p.B, p.Lq, p.Lk, p.Hq, p.Hkv, true)) ns = 1;
  float* part_out = nullptr;
  float* part_lse = nullptr;
  if (ns > 1) {
    char* parts = w + align256((size_t)nflags * sizeof(int)) + align256(ody_attn_images_bytes(p.B, p.Lk, p.Hkv));
    part_out = reinterpret_cast<float*>(parts);
    part_lse = reinterpret_cast<float*>(parts + align256((size_t)ns * p.B * p.Lq * p.Hq * D * sizeof(float)));
  }
  dim3 grid(nqb * p.Hq * p.B * ns);
  ODY_LAUNCH("attn_fwd_w8", st, attn_fwd_w8_kernel, grid, dim3(FW_THREADS), smem, p, images, flags, ns, part_out, part_lse);
  rc = ody_check_launch("attn_fwd_w8");
  if (rc) return rc;
  if (ns > 1) {
    const int64_t n4 = (int64_t)p.B * p.Lq * p.Hq * (D / 4);
    ODY_LAUNCH("attn_fwd_split_merge", st, attn_fwd_split_merge_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, p, ns,
               part_out, part_lse);
    if ((rc = ody_check_launch("attn_fwd_split_merge"))) return rc;
  }
  return ody_launch_attn_fwd_mfma_flagged(p, flags, FW_BM, st);
}
