// Causal / full flash-attention forward for gfx950, bf16 in, fp32 accumulate.
//
// Work split: one workgroup (4 wavefronts) owns BM = 4 * 32 * QT consecutive
// query rows of one (batch, head); each wavefront owns 32 * QT of them and
// streams the keys in tiles of BN = 64 through LDS (double-buffered, filled
// with 16-byte global loads that are issued one tile ahead).
//
// Both contractions are computed TRANSPOSED so that every per-query quantity
// (running max, running sum, rescale factor, lse) is constant within a lane:
//
//   S^T (keys x queries) = K (keys x d) . Q^T (d x queries)
//        A operand: K rows straight from LDS (16-byte reads),
//        B operand: this lane's query row, held in registers for the whole kernel.
//   O^T (d x queries)   += V^T (d x keys) . P^T (keys x queries)
//        B operand: P^T is exactly the accumulator layout of S^T (a lane holds
//        8 consecutive-in-k values per k-step), so P never leaves registers;
//        A operand: V^T read from the row-major V tile with the LDS transpose
//        read (ds_read_b64_tr_b16).
//
// v_mfma_f32_32x32x16_bf16 layouts (lane = 32*g + i):
//   A: row i, k = 8g..8g+7      B: column i, k = 8g..8g+7
//   C: column i, rows 8*(r/4) + 4g + r%4 for register r = 0..15
#include "attn_params.h"

namespace {

// DROP: attention dropout (AttnParams::drop_*): the row sums, and with them lse, are those of the full P; the entries
// that go into P . V are the kept ones, and the result is scaled by 1 / (1 - p) at the end.
template <int D, int QT, bool DROP>
__global__ __launch_bounds__(256, 2) void attn_fwd_mfma_kernel(const AttnParams p, const int* __restrict__ flags,
                                                               int flag_block) {
  constexpr int BN = 64, WQ = 32 * QT, BM = 4 * WQ;
  constexpr int KP = D + 8;    // K tile row pitch (elements): 16-byte reads of 16 rows hit 64 distinct banks
  constexpr int VP = D + 32;   // V tile row pitch: 4 rows x 32 columns of a transpose read hit distinct banks
  constexpr int KS = D / 16, DT = D / 32;
  constexpr int CPR = D / 8;                // 16-byte chunks per tile row
  constexpr int CHUNKS = BN * CPR / 256;    // chunks per thread per tile

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* Ks = reinterpret_cast<bf16*>(smem_raw);            // [2][BN][KP]
  bf16* Vs = Ks + 2 * BN * KP;                             // [2][BN][VP]

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 5, i = lane & 31;
  const BlockCoord bc = ody_block_coord(p.Hq, p.B);
  const int nqb = gridDim.x / (p.Hq * p.B);
  const int qblk = p.causal ? (nqb - 1 - bc.rank) : bc.rank;   // heaviest blocks first
  const int h = bc.h, b = bc.b, hk = h / p.group;
  const int q0 = qblk * BM, wq0 = q0 + wave * WQ;
  // restricted run: only query blocks whose flag is set (the flags cover blocks of flag_block rows)
  if (flags != nullptr) {
    const int nfb = (p.Lq + flag_block - 1) / flag_block;
    if (flags[((int64_t)b * p.Hq + h) * nfb + q0 / flag_block] == 0) return;
  }

  const bf16* qp = static_cast<const bf16*>(p.q) + b * p.sq.b + h * p.sq.h;
  const bf16* kp = static_cast<const bf16*>(p.k) + b * p.sk.b + hk * p.sk.h;
  const bf16* vp = static_cast<const bf16*>(p.v) + b * p.sv.b + hk * p.sv.h;

  // ---- this lane's query rows as B operands
  bf16x8 qf[QT][KS];
#pragma unroll
  for (int qt = 0; qt < QT; qt++) {
    const int qi = wq0 + 32 * qt + i;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (qi < p.Lq) qf[qt][ks] = *reinterpret_cast<const bf16x8*>(qp + (int64_t)qi * p.sq.l + 16 * ks + 8 * g);
      else qf[qt][ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }

  f32x16 o[QT][DT];
  float m[QT], l[QT];
#pragma unroll
  for (int qt = 0; qt < QT; qt++) {
    m[qt] = -INFINITY;
    l[qt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[qt][dt][r] = 0.f;
  }

  const int q_hi = min(q0 + BM, p.Lq) - 1;
  int n_end = p.causal ? min(p.Lk, q_hi + p.off + 1) : p.Lk;
  if (n_end < 0) n_end = 0;
  const int ntiles = (n_end + BN - 1) / BN;

  bf16x8 kr[CHUNKS], vr[CHUNKS];
  auto gload = [&](int n0) {
#pragma unroll
    for (int j = 0; j < CHUNKS; j++) {
      const int c = tid + 256 * j, row = c / CPR, col = (c % CPR) * 8, key = n0 + row;
      if (key < p.Lk) {
        kr[j] = *reinterpret_cast<const bf16x8*>(kp + (int64_t)key * p.sk.l + col);
        vr[j] = *reinterpret_cast<const bf16x8*>(vp + (int64_t)key * p.sv.l + col);
      } else {
        kr[j] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
        vr[j] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
  };
  auto sstore = [&](int buf) {
#pragma unroll
    for (int j = 0; j < CHUNKS; j++) {
      const int c = tid + 256 * j, row = c / CPR, col = (c % CPR) * 8;
      *reinterpret_cast<bf16x8*>(Ks + (buf * BN + row) * KP + col) = kr[j];
      *reinterpret_cast<bf16x8*>(Vs + (buf * BN + row) * VP + col) = vr[j];
    }
  };

  if (ntiles > 0) {
    gload(0);
    sstore(0);
  }
  __syncthreads();

  const float c2 = p.scale_log2e;
  unsigned drow[QT];
  if (DROP) {
    const unsigned dh = ody_dropout_head(p.drop_seed, b * p.Hq + h);
#pragma unroll
    for (int qt = 0; qt < QT; qt++) drow[qt] = ody_dropout_row(dh, wq0 + 32 * qt + i);
  }
  // transpose-read addressing inside a 16-lane block
  const int tr_row = (i & 15) >> 2, tr_col = 16 * (i >> 4) + 4 * (i & 3);

  for (int t = 0; t < ntiles; t++) {
    const int buf = t & 1, n0 = t * BN;
    if (t + 1 < ntiles) gload(n0 + BN);

    const bool active = !p.causal || (n0 <= wq0 + WQ - 1 + p.off);
    if (active) {
      const bf16* Kb = Ks + buf * BN * KP;
      const bf16* Vb = Vs + buf * BN * VP;
      // ---- S^T = K . Q^T
      f32x16 s[QT][2];
#pragma unroll
      for (int qt = 0; qt < QT; qt++)
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
          for (int r = 0; r < 16; r++) s[qt][kt][r] = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          const bf16x8 a = *reinterpret_cast<const bf16x8*>(Kb + (32 * kt + i) * KP + 16 * ks + 8 * g);
#pragma unroll
          for (int qt = 0; qt < QT; qt++) s[qt][kt] = mfma32(a, qf[qt][ks], s[qt][kt]);
        }
      }
      // ---- mask
      const bool need_mask = (n0 + BN > p.Lk) || (p.causal && (n0 + BN - 1 > wq0 + p.off));
      if (need_mask) {
#pragma unroll
        for (int qt = 0; qt < QT; qt++) {
          const int lim = p.causal ? min(p.Lk - 1, wq0 + 32 * qt + i + p.off) : p.Lk - 1;
#pragma unroll
          for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
              const int key = n0 + 32 * kt + 8 * (r >> 2) + 4 * g + (r & 3);
              if (key > lim) s[qt][kt][r] = -INFINITY;
            }
        }
      }
      // ---- online softmax (per query = per lane pair {i, i+32})
      bf16x8 pb[QT][2][2];
#pragma unroll
      for (int qt = 0; qt < QT; qt++) {
        float mx = s[qt][0][0];
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
          for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[qt][kt][r]);
        mx = fmaxf(mx, xor32(mx));
        const float m_new = fmaxf(m[qt], mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = ody_exp2((m[qt] - m_use) * c2);
        const float mc = m_use * c2;
        m[qt] = m_new;
        float rs = 0.f;
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const float e = ody_exp2(fmaf(s[qt][kt][r], c2, -mc));
            s[qt][kt][r] = e;
            rs += e;
          }
        l[qt] = l[qt] * alpha + rs;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
          for (int r = 0; r < 16; r++) o[qt][dt][r] *= alpha;
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
          for (int ss = 0; ss < 2; ss++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
              float x = s[qt][kt][8 * ss + e];
              if (DROP) {
                const int r = 8 * ss + e, key = n0 + 32 * kt + 8 * (r >> 2) + 4 * g + (r & 3);
                if (ody_dropout_hash(drow[qt], key) < p.drop_thresh) x = 0.f;
              }
              pb[qt][kt][ss][e] = (bf16)x;
            }
      }
      // ---- O^T += V^T . P^T
#pragma unroll
      for (int dt = 0; dt < DT; dt++) {
#pragma unroll
        for (int kt = 0; kt < 2; kt++) {
#pragma unroll
          for (int ss = 0; ss < 2; ss++) {
            const int kbase = 32 * kt + 16 * ss + 4 * g;
            const bf16* vptr = Vb + (kbase + tr_row) * VP + 32 * dt + tr_col;
            const bf16x8 a = concat4(lds_read_tr16(vptr), lds_read_tr16(vptr + 8 * VP));
#pragma unroll
            for (int qt = 0; qt < QT; qt++) o[qt][dt] = mfma32(a, pb[qt][kt][ss], o[qt][dt]);
          }
        }
      }
    }
    if (t + 1 < ntiles) sstore(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue
  bf16* op = static_cast<bf16*>(p.out) + b * p.so.b + h * p.so.h;
  float* lsep = p.lse + ((int64_t)b * p.Hq + h) * p.Lq;
#pragma unroll
  for (int qt = 0; qt < QT; qt++) {
    const int qi = wq0 + 32 * qt + i;
    const float lt = l[qt] + xor32(l[qt]);
    const float inv = lt > 0.f ? (DROP ? p.drop_scale : 1.f) / lt : 0.f;
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
      if (g == 0) lsep[qi] = lt > 0.f ? m[qt] * p.scale + __logf(lt) : -INFINITY;
    }
  }
}

template <int D, int QT, bool DROP>
int launch(const AttnParams& p, const int* flags, int flag_block, hipStream_t st) {
  constexpr int BN = 64, BM = 4 * 32 * QT;
  constexpr size_t smem = (size_t)2 * BN * ((D + 8) + (D + 32)) * sizeof(bf16);
  if (int rc = ody_allow_dynamic_lds(reinterpret_cast<const void*>(&attn_fwd_mfma_kernel<D, QT, DROP>), smem, "attn_fwd"))
    return rc;
  dim3 grid(((p.Lq + BM - 1) / BM) * p.Hq * p.B);
  ODY_LAUNCH("attn_fwd_mfma", st, (attn_fwd_mfma_kernel<D, QT, DROP>), grid, dim3(256), smem, p, flags, flag_block);
  return ody_check_launch("attn_fwd_mfma");
}

}  // namespace

int ody_launch_attn_fwd_mfma(const AttnParams& p, int D, hipStream_t st) {
  if (p.drop_thresh != 0) {
    if (D == 128) return launch<128, 1, true>(p, nullptr, 1, st);
    if (D == 64) return launch<64, 1, true>(p, nullptr, 1, st);
  } else {
    if (D == 128) return launch<128, 1, false>(p, nullptr, 1, st);
    if (D == 64) return launch<64, 1, false>(p, nullptr, 1, st);
  }
  ody_set_error("attn_fwd: head_dim %d not built (64, 128)", D);
  return ODY_ERR_UNSUPPORTED;
}

int ody_launch_attn_fwd_mfma_flagged(const AttnParams& p, const int* flags, int block, hipStream_t st) {
  return launch<128, 1, false>(p, flags, block, st);
}
