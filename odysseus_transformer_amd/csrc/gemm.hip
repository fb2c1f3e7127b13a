// Dense linears: C (M, N) = op(A) . op(B) for the three products of a linear
// layer (forward NT, dgrad NN, wgrad TN).
//
// bf16: v_mfma_f32_32x32x16_bf16, 4 wavefronts in a 2 x 2 arrangement, each
// owning WM x WN accumulator tiles of 32 x 32; operands are staged through LDS
// in K-slabs of 64, double-buffered, filled with 16-byte global loads issued one
// slab ahead.  An operand whose memory is contiguous along K is kept as
// [rows][64 + 8] and read with 16-byte row reads; one that is contiguous along
// M or N is kept as [64][cols + 32] and read with the LDS transpose read, so no
// operand is ever transposed in global memory.  The product is computed as
// C^T = op(B)^T . op(A)^T so that a lane ends up with 4 consecutive N per
// register quad and writes 8-byte pieces of C rows.
//
// fp32 (its 1e-4 tolerance rules out bf16 inputs): v_mfma_f32_32x32x2_f32 on
// 64 x 64 or 128 x 128 workgroup tiles, any shape and alignment.
#include <type_traits>
#include "ody_common.h"

namespace {

// ------------------------------------------------------------------ bf16 MFMA
constexpr int BK = 64;

// Operand tile in LDS.  KC = true: memory is (rows, K) row-major -> [ROWS][BK+8].
//                       KC = false: memory is (K, rows) row-major -> [BK][ROWS+32].
template <int ROWS, bool KC>
struct OperandTile {
  static constexpr int PITCH = KC ? (BK + 8) : (ROWS + 32);
  static constexpr int ELEMS = KC ? ROWS * PITCH : BK * PITCH;
  static constexpr int CHUNKS = ROWS * BK / 8 / 256;  // 16-byte chunks per thread
  bf16x8 r[CHUNKS];

  // row0: first row (M or N index) of the tile; k0: first K index
  __device__ __forceinline__ void gload(const bf16* base, int64_t ld, int row0, int k0, int nrows, int K, int tid) {
#pragma unroll
    for (int j = 0; j < CHUNKS; j++) {
      const int c = tid + 256 * j;
      int rr, kk;
      if (KC) { rr = c / (BK / 8); kk = (c % (BK / 8)) * 8; }
      else { kk = c / (ROWS / 8); rr = (c % (ROWS / 8)) * 8; }
      const int gr = row0 + rr, gk = k0 + kk;
      bool ok;
      const bf16* src;
      if (KC) { ok = gr < nrows && gk < K; src = base + (int64_t)gr * ld + gk; }   // K % 8 == 0: chunk all in or out
      else { ok = gk < K && gr < nrows; src = base + (int64_t)gk * ld + gr; }      // rows % 8 == 0 likewise
      r[j] = ok ? *reinterpret_cast<const bf16x8*>(src) : bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  __device__ __forceinline__ void sstore(bf16* lds, int tid) const {
#pragma unroll
    for (int j = 0; j < CHUNKS; j++) {
      const int c = tid + 256 * j;
      int rr, kk;
      if (KC) { rr = c / (BK / 8); kk = (c % (BK / 8)) * 8; *reinterpret_cast<bf16x8*>(lds + rr * PITCH + kk) = r[j]; }
      else { kk = c / (ROWS / 8); rr = (c % (ROWS / 8)) * 8; *reinterpret_cast<bf16x8*>(lds + kk * PITCH + rr) = r[j]; }
    }
  }
  // MFMA operand for tile rows [r32, r32+32), k-step ks (16 K values): lane (g, i) gets row r32+i, k = 16ks+8g..+7
  __device__ static __forceinline__ bf16x8 frag(const bf16* lds, int r32, int ks, int g, int i) {
    if (KC) {
      return *reinterpret_cast<const bf16x8*>(lds + (r32 + i) * PITCH + 16 * ks + 8 * g);
    } else {
      const bf16* p = lds + (16 * ks + 8 * g + ((i & 15) >> 2)) * PITCH + r32 + 16 * (i >> 4) + 4 * (i & 3);
      return concat4(lds_read_tr16(p), lds_read_tr16(p + 4 * PITCH));
    }
  }
  // The same for the 16 x 16 x 32 MFMA: tile rows [r16, r16 + 16), k-step ks (32 K values): lane l gets row
  // r16 + (l & 15), k = 32 ks + 8 (l >> 4) .. + 7
  __device__ static __forceinline__ bf16x8 frag16(const bf16* lds, int r16, int ks, int lane) {
    const int c = lane & 15, q = lane >> 4;
    if (KC) {
      return *reinterpret_cast<const bf16x8*>(lds + (r16 + c) * PITCH + 32 * ks + 8 * q);
    } else {
      const bf16* p = lds + (32 * ks + 8 * q + (c >> 2)) * PITCH + r16 + 4 * (c & 3);
      return concat4(lds_read_tr16(p), lds_read_tr16(p + 4 * PITCH));
    }
  }
};

// Interior tiles with K a multiple of 64 take this kernel.  Same tiles and fragments as the
// general kernel below, but the traffic of the next slabs is spread over the MFMA stream
// instead of being issued in bursts: a wavefront is held up while the memory pipeline accepts
// its loads (64 bytes per clock per CU) and while the LDS takes its writes, and with one
// wavefront per SIMD the matrix pipe idles meanwhile.  Per 16-MFMA k-step the wavefront writes
// a quarter of its staging registers (slab kt+1, loaded one iteration earlier) to the other LDS
// buffer, refills them at once with their part of slab kt+2, and reads the fragments of the next
// k-step.
#define GEMM_FENCE() __builtin_amdgcn_sched_barrier(0)

// 16 bytes of a result row on their way out, as a streaming store: this kernel does not read them again (products
// with a large output for their K gain 3-5 % when timed alone -- QKV and gate_up forward, O dgrad --, the layer as a
// whole neither gains nor loses: its next kernel then reads the rows from memory instead of from cache)
__device__ __forceinline__ void store_out16(bf16* dst, bf16x8 w) {
  typedef unsigned raw_t __attribute__((ext_vector_type(4)));
  __builtin_nontemporal_store(__builtin_bit_cast(raw_t, w), reinterpret_cast<raw_t*>(dst));
}

// What the fast kernel's epilogue does besides rounding and storing the tile.
//   EPI_RESIDUAL    C = A B + R                      (R = aux, row pitch ld_aux; one rounding, after the add)
//   EPI_SWIGLU_FWD  NT only.  B is the packed (2 I, K) gate_up weight.  A 256-column tile holds 128 gate columns
//                   and the 128 matching up columns, interleaved in blocks of 32 (block c of the tile: gate if c is
//                   even, up if odd, columns j0 + 32 (c / 2) ...), so that a lane owns gate and up of the same
//                   (token, j).  Writes gate_up to C in its usual [gate | up] layout and h = silu(gate) * up to out2,
//                   computed from the rounded gate / up values exactly as the stand-alone SwiGLU kernel would.
//   EPI_ROPE        NT only, head_dim 128.  A wavefront's 128 columns are one head; columns below I (a multiple of 128)
//                   are rotated before the one rounding: with the cos / sin table of ody_rope_table in aux (row pitch
//                   ld_aux), column j < 64 of a head pairs with column j + 64, both in the same lane
//   EPI_SWIGLU_BWD  the tile is dh = dy Wd (N = I); with gate_up = aux the epilogue writes d_gate_up to C (pitch
//                   ldc, 2 I columns) as the stand-alone SwiGLU backward would from the rounded dh.
enum { EPI_NONE = 0, EPI_RESIDUAL = 1, EPI_SWIGLU_FWD = 2, EPI_SWIGLU_BWD = 3, EPI_ROPE = 4 };
struct GemmEpi {
  const bf16* aux;
  bf16* out2;
  int64_t ld_aux, ld_out2;
  int I;
};

//
// SPLITK: blockIdx.y selects one of gridDim.y ranges of K slabs; the block writes its fp32 partial tile to
// part[blockIdx.y][M][N] and gemm_splitk_sum_kernel adds the ranges up (bias, C += and the rounding happen
// there).  For products with a long K and few output tiles (weight gradients) this is what fills the chip.
template <int WM, int WN, bool A_KC, bool B_KC, bool SPLITK, int EPI = EPI_NONE>
__global__ __launch_bounds__(256) void gemm_bf16_fast_kernel(const bf16* __restrict__ A, const bf16* __restrict__ B,
                                                             bf16* __restrict__ C, const bf16* __restrict__ bias,
                                                             int M, int N, int K, int64_t lda, int64_t ldb,
                                                             int64_t ldc, int accumulate, int tiles_m, int tiles_n,
                                                             float* __restrict__ part, GemmEpi ep) {
  static_assert(EPI == EPI_NONE || (!SPLITK && WM == 4 && WN == 4), "fused epilogues: 256 x 256 tiles, one pass over K");
  static_assert(EPI != EPI_SWIGLU_FWD || (A_KC && B_KC), "the SwiGLU forward epilogue belongs to the NT product");
  static_assert(EPI != EPI_ROPE || (A_KC && B_KC), "the rotary epilogue belongs to the NT product");
  constexpr int TM = 64 * WM, TN = 64 * WN;
  typedef OperandTile<TM, A_KC> TA;
  typedef OperandTile<TN, B_KC> TB;
  constexpr int CA = TA::CHUNKS, CB = TB::CHUNKS, KSTEPS = BK / 16;
  static_assert(CA % KSTEPS == 0 && CB % KSTEPS == 0, "chunks are issued a quarter per k-step");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* As = reinterpret_cast<bf16*>(smem_raw);  // [2][TA::ELEMS]
  bf16* Bs = As + 2 * TA::ELEMS;                 // [2][TB::ELEMS]

  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, g = lane >> 5,
            i = lane & 31;
  const int wm = wave >> 1, wn = wave & 1;

  int pid = blockIdx.x;
  const int nblk = tiles_m * tiles_n;
  if (nblk % 8 == 0) pid = (pid % 8) * (nblk / 8) + pid / 8;
  constexpr int GROUP = 8;
  const int per_group = GROUP * tiles_n;
  const int gid = pid / per_group, first_m = gid * GROUP;
  const int gsz = min(tiles_m - first_m, GROUP);
  const int tm = first_m + (pid % per_group) % gsz, tn = (pid % per_group) / gsz;
  const int m0 = tm * TM, n0 = tn * TN;

  // chunk j of a thread: global element offset = off0 + j * step (+ slab advance), LDS element offset = lds0 + j * lstep
  unsigned a_off0, b_off0, a_lds0, b_lds0;
  int64_t a_step, b_step, a_slab, b_slab;
  int a_lstep, b_lstep;
  if (A_KC) {
    a_off0 = (unsigned)((tid / 8) * lda + (tid % 8) * 8); a_step = 32 * lda; a_slab = BK;
    a_lds0 = (tid / 8) * TA::PITCH + (tid % 8) * 8; a_lstep = 32 * TA::PITCH;
  } else {
    a_off0 = (unsigned)((tid / (TM / 8)) * lda + (tid % (TM / 8)) * 8); a_step = (256 / (TM / 8)) * lda; a_slab = BK * lda;
    a_lds0 = (tid / (TM / 8)) * TA::PITCH + (tid % (TM / 8)) * 8; a_lstep = (256 / (TM / 8)) * TA::PITCH;
  }
  if (B_KC) {
    b_off0 = (unsigned)((tid / 8) * ldb + (tid % 8) * 8); b_step = 32 * ldb; b_slab = BK;
    b_lds0 = (tid / 8) * TB::PITCH + (tid % 8) * 8; b_lstep = 32 * TB::PITCH;
  } else {
    b_off0 = (unsigned)((tid / (TN / 8)) * ldb + (tid % (TN / 8)) * 8); b_step = (256 / (TN / 8)) * ldb; b_slab = BK * ldb;
    b_lds0 = (tid / (TN / 8)) * TB::PITCH + (tid % (TN / 8)) * 8; b_lstep = (256 / (TN / 8)) * TB::PITCH;
  }
  // this block's range of K slabs
  int nk = K / BK, kt0 = 0;
  if (SPLITK) {
    const int per = (nk + (int)gridDim.y - 1) / (int)gridDim.y;
    kt0 = blockIdx.y * per;
    nk = max(0, min(nk - kt0, per));
  }
  const bf16* Abase = (A_KC ? A + (int64_t)m0 * lda : A + m0) + (int64_t)kt0 * a_slab;   // first element of the first slab
  // EPI_SWIGLU_FWD: tile tn covers j in [128 tn, 128 tn + 128); chunk j of a thread lies in the tile's 32-row block j
  const bf16* Bbase = (EPI == EPI_SWIGLU_FWD ? B + (int64_t)(n0 / 2) * ldb : (B_KC ? B + (int64_t)n0 * ldb : B + n0)) +
                      (int64_t)kt0 * b_slab;
  const int64_t b_up = (int64_t)ep.I * ldb;   // from a gate row to its up row

  // The 16 x 16 x 32 instruction does the same work for less energy (a register-only loop sustains 12-14 % more with
  // it at the package power limit); measured inside this kernel it is worth +3 % where both the main loop and the
  // epilogue keep within the register file: 256 x 256 tiles, A contiguous along K, one pass over K, and not the
  // SwiGLU epilogues.  Those instances run the main loop on 2 WM x 2 WN tiles of 16 x 16 and bring one band of
  // accumulators at a time into the 32 x 32 layout that the epilogues are written for.
  constexpr bool M16 = WM == 4 && WN == 4 && A_KC && !SPLITK && (EPI == EPI_NONE || EPI == EPI_RESIDUAL || EPI == EPI_ROPE);
  f32x16 acc[M16 ? 1 : WM][M16 ? 1 : WN];
  f32x4 acc16[M16 ? 2 * WM : 1][M16 ? 2 * WN : 1];
  if constexpr (M16) {
#pragma unroll
    for (int a = 0; a < 2 * WM; a++)
#pragma unroll
      for (int b = 0; b < 2 * WN; b++) acc16[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  } else {
#pragma unroll
    for (int a = 0; a < WM; a++)
#pragma unroll
      for (int b = 0; b < WN; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;
  }

  bf16x8 ra[CA], rb[CB];
  auto gload_a = [&](int kt, int j) {
    ra[j] = *reinterpret_cast<const bf16x8*>(Abase + (int64_t)kt * a_slab + j * a_step + a_off0);
  };
  auto gload_b = [&](int kt, int j) {
    const int64_t rows = EPI == EPI_SWIGLU_FWD ? (j & 1) * b_up + (j >> 1) * b_step : j * b_step;
    rb[j] = *reinterpret_cast<const bf16x8*>(Bbase + (int64_t)kt * b_slab + rows + b_off0);
  };
  auto sstore_a = [&](int buf, int j) { *reinterpret_cast<bf16x8*>(As + buf * TA::ELEMS + a_lds0 + j * a_lstep) = ra[j]; };
  auto sstore_b = [&](int buf, int j) { *reinterpret_cast<bf16x8*>(Bs + buf * TB::ELEMS + b_lds0 + j * b_lstep) = rb[j]; };

  if (nk > 0) {
#pragma unroll
  for (int j = 0; j < CA; j++) gload_a(0, j);
#pragma unroll
  for (int j = 0; j < CB; j++) gload_b(0, j);
#pragma unroll
  for (int j = 0; j < CA; j++) sstore_a(0, j);
#pragma unroll
  for (int j = 0; j < CB; j++) sstore_b(0, j);
  {
    // in the order in which the main loop re-issues them (A and B chunks alternating): the compiler sizes the
    // loop's s_waitcnt vmcnt for the oldest order it can see, and with all A loads ahead of all B loads here it
    // made every B chunk's LDS store wait for loads issued half a slab ago instead of a whole one
    const int k1 = min(1, nk - 1);
    static_assert(CA == CB, "chunks alternate");
#pragma unroll
    for (int j = 0; j < CA; j++) {
      gload_a(k1, j);
      GEMM_FENCE();   // or the scheduler clusters the loads by base pointer again
      gload_b(k1, j);
      GEMM_FENCE();
    }
  }
  }
  __syncthreads();

  // Slab kt is in LDS buffer kt & 1 and the registers hold slab kt+1.  During the first KSTEPS - 1 k-steps
  // of a slab the staging registers go, one or two 16-byte chunks per group of WN MFMAs, to the other LDS
  // buffer and are refilled at once with their part of slab kt+2.  The one barrier of the slab sits INSIDE
  // the last k-step, behind its first group of MFMAs: by then every wavefront has written its part of slab
  // kt+1 and has read its last fragments of slab kt, so the fragments of slab kt+1's first k-step can be
  // fetched under the remaining MFMAs of slab kt instead of in front of an idle matrix pipe.
  if constexpr (M16) {
    // The main loop on v_mfma_f32_16x16x32_bf16: 2 WM x 2 WN accumulator tiles of 16 x 16, two k-steps of 32 per slab;
    // same LDS layout, same staging schedule.  The accumulators are brought into the 32 x 32 layout afterwards.
    static_assert(CA == CB, "chunk schedule");
    constexpr int WM2 = 2 * WM, WN2 = 2 * WN, KS2 = BK / 32;
    static_assert(KS2 == 2 && WM2 == WN2, "fragment sets alternate per k-step");
    constexpr int MOVES = CA + CB, GROUPS = (KS2 - 1) * WM2;
    bf16x8 af[2][WM2], bfr[2][WN2];
    if (nk > 0) {
#pragma unroll
      for (int a = 0; a < WM2; a++) af[0][a] = TA::frag16(As, 16 * (wm * WM2 + a), 0, lane);
#pragma unroll
      for (int b = 0; b < WN2; b++) bfr[0][b] = TB::frag16(Bs, 16 * (wn * WN2 + b), 0, lane);
    }
    for (int kt = 0; kt < nk; kt++) {
      const int buf = kt & 1;
      const bf16* Ab = As + buf * TA::ELEMS;
      const bf16* Bb = Bs + buf * TB::ELEMS;
      const bf16* An = As + (buf ^ 1) * TA::ELEMS;
      const bf16* Bn = Bs + (buf ^ 1) * TB::ELEMS;
      const int kt2 = min(kt + 2, nk - 1);   // past the end: a harmless re-load, and a write nobody reads
      GEMM_FENCE();
#pragma unroll
      for (int ks = 0; ks < KS2; ks++) {
        const int cur = ks & 1, nxt = cur ^ 1;
#pragma unroll
        for (int a = 0; a < WM2; a++) {
#pragma unroll
          for (int b = 0; b < WN2; b++)
            acc16[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bfr[cur][b], af[cur][a], acc16[a][b], 0, 0, 0);   // rows = n, cols = m
          if (ks + 1 < KS2) {
            af[nxt][a] = TA::frag16(Ab, 16 * (wm * WM2 + a), ks + 1, lane);
            bfr[nxt][a] = TB::frag16(Bb, 16 * (wn * WN2 + a), ks + 1, lane);
            const int gi = ks * WM2 + a;
#pragma unroll
            for (int m = gi * MOVES / GROUPS; m < (gi + 1) * MOVES / GROUPS; m++) {
              if (m % 2 == 0) { sstore_a(buf ^ 1, m / 2); gload_a(kt2, m / 2); }
              else { sstore_b(buf ^ 1, m / 2); gload_b(kt2, m / 2); }
            }
          } else {
            if (a == 0) __syncthreads();
            af[nxt][a] = TA::frag16(An, 16 * (wm * WM2 + a), 0, lane);
            bfr[nxt][a] = TB::frag16(Bn, 16 * (wn * WN2 + a), 0, lane);
          }
          GEMM_FENCE();
        }
      }
    }
  } else {
    static_assert(CA == CB && KSTEPS > 1, "chunk schedule");
    constexpr int MOVES = CA + CB, GROUPS = (KSTEPS - 1) * WM;
    bf16x8 af[2][WM], bfr[2][WN];
    if (nk > 0) {
#pragma unroll
      for (int a = 0; a < WM; a++) af[0][a] = TA::frag(As, 32 * (wm * WM + a), 0, g, i);
#pragma unroll
      for (int b = 0; b < WN; b++) bfr[0][b] = TB::frag(Bs, 32 * (wn * WN + b), 0, g, i);
    }
    for (int kt = 0; kt < nk; kt++) {
      const int buf = kt & 1;
      const bf16* Ab = As + buf * TA::ELEMS;
      const bf16* Bb = Bs + buf * TB::ELEMS;
      const bf16* An = As + (buf ^ 1) * TA::ELEMS;
      const bf16* Bn = Bs + (buf ^ 1) * TB::ELEMS;
      const int kt2 = min(kt + 2, nk - 1);   // past the end: a harmless re-load, and a write nobody reads
      GEMM_FENCE();
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) {
        const int cur = ks & 1, nxt = cur ^ 1;
#pragma unroll
        for (int a = 0; a < WM; a++) {
#pragma unroll
          for (int b = 0; b < WN; b++) acc[a][b] = mfma32(bfr[cur][b], af[cur][a], acc[a][b]);  // rows = n, cols = m
          if (ks + 1 < KSTEPS) {
            af[nxt][a] = TA::frag(Ab, 32 * (wm * WM + a), ks + 1, g, i);
            if (a < WN) bfr[nxt][a] = TB::frag(Bb, 32 * (wn * WN + a), ks + 1, g, i);
            const int gi = ks * WM + a;
#pragma unroll
            for (int m = gi * MOVES / GROUPS; m < (gi + 1) * MOVES / GROUPS; m++) {
              if (m % 2 == 0) { sstore_a(buf ^ 1, m / 2); gload_a(kt2, m / 2); }
              else { sstore_b(buf ^ 1, m / 2); gload_b(kt2, m / 2); }
            }
          } else {
            if (a == 0) __syncthreads();
            // first fragments of the next slab (KSTEPS is even: they land in set 0)
            af[nxt][a] = TA::frag(An, 32 * (wm * WM + a), 0, g, i);
            if (a < WN) bfr[nxt][a] = TB::frag(Bn, 32 * (wn * WN + a), 0, g, i);
          }
          GEMM_FENCE();
        }
      }
    }
  }
  __syncthreads();   // the epilogue (and the conversion in front of it) reuse the operand buffers
  // lane l holds column m = l & 15 and rows n = 4 (l >> 4) + r of each 16 x 16 tile; the epilogues expect column
  // m = l & 31 and rows n = 8 (r / 4) + 4 (l >> 5) + r % 4 of each 32 x 32 tile.  One band of WN tiles at a time
  // makes a round trip through a private fp32 patch (a wavefront's LDS operations complete in order).
  constexpr int CP = 36;
  float* conv = reinterpret_cast<float*>(smem_raw) + 4 * 32 * (32 * WN + 4) + wave * 32 * CP;
  static_assert(!M16 || (4 * 32 * (32 * WN + 4) + 4 * 32 * CP) * 4 <= 2 * (TA::ELEMS + TB::ELEMS) * 2, "the patches fit behind the bands");
  f32x16 acc_row[WN];
  auto load_row = [&](int a) {
    if constexpr (!M16) return;
    const int c = lane & 15, q4 = lane >> 4;
#pragma unroll
    for (int b = 0; b < WN; b++) {
#pragma unroll
      for (int ta = 0; ta < 2; ta++)
#pragma unroll
        for (int tb = 0; tb < 2; tb++)
          *reinterpret_cast<f32x4*>(conv + (16 * ta + c) * CP + 16 * tb + 4 * q4) = acc16[2 * a + ta][2 * b + tb];
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(conv + i * CP + 8 * q + 4 * g);
#pragma unroll
        for (int e = 0; e < 4; e++) acc_row[b][4 * q + e] = v[e];
      }
    }
  };
  auto acc_tile = [&](int a, int b) -> const f32x16& {
    if constexpr (M16) return acc_row[b];
    else return acc[a][b];
  };
#define ACC(a, b) acc_tile(a, b)
#define LOAD_ROW(a) load_row(a)

  // Epilogue.  Lane (g, i) holds column m = i and rows n = 8*(r/4) + 4g + r%4 of each 32 x 32 tile,
  // i.e. 8-byte pieces of 32 different rows of C.  Unless C is accumulated into, the tiles go
  // through LDS (free by now) one 32-row band at a time and leave as 16-byte pieces of whole rows.
  if (SPLITK) {
    // fp32 partial tile, through LDS like below: 32-row bands, 16-byte pieces of whole rows
    constexpr int EPF = 32 * WN + 4;
    float* band = reinterpret_cast<float*>(smem_raw) + wave * 32 * EPF;
    static_assert(4 * 32 * EPF * 2 <= 2 * (TA::ELEMS + TB::ELEMS), "the fp32 bands fit in the operand buffers");
    float* dst0 = part + ((int64_t)blockIdx.y * M + m0) * N + n0 + 32 * wn * WN;
#pragma unroll
    for (int a = 0; a < WM; a++) {
    LOAD_ROW(a);
#pragma unroll
      for (int b = 0; b < WN; b++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          f32x4 v;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = ACC(a, b)[4 * q + e];
          *reinterpret_cast<f32x4*>(band + i * EPF + 32 * b + 8 * q + 4 * g) = v;
        }
      constexpr int CPR = 32 * WN / 4, RPP = 64 / CPR;                  // 16-byte chunks per row, rows per pass
#pragma unroll
      for (int pass = 0; pass < 32 / RPP; pass++) {
        const int row = pass * RPP + lane / CPR, c = lane % CPR;
        const f32x4 v = *reinterpret_cast<const f32x4*>(band + row * EPF + 4 * c);
        *reinterpret_cast<f32x4*>(dst0 + (int64_t)(32 * (wm * WM + a) + row) * N + 4 * c) = v;
      }
    }
    return;
  }
  if constexpr (EPI == EPI_RESIDUAL) {
    // fp32 bands, so that the residual is added before the one rounding; 16-byte pieces of whole rows of R and C
    constexpr int EPF = 32 * WN + 4;
    float* band = reinterpret_cast<float*>(smem_raw) + wave * 32 * EPF;
    static_assert(4 * 32 * EPF * 2 <= 2 * (TA::ELEMS + TB::ELEMS), "the fp32 bands fit in the operand buffers");
#pragma unroll
    for (int a = 0; a < WM; a++) {
    LOAD_ROW(a);
#pragma unroll
      for (int b = 0; b < WN; b++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          f32x4 v;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = ACC(a, b)[4 * q + e];
          *reinterpret_cast<f32x4*>(band + i * EPF + 32 * b + 8 * q + 4 * g) = v;
        }
      constexpr int CPR = 32 * WN / 8, RPP = 64 / CPR;
#pragma unroll
      for (int pass = 0; pass < 32 / RPP; pass++) {
        const int row = pass * RPP + lane / CPR, c = lane % CPR;
        const f32x4 v0 = *reinterpret_cast<const f32x4*>(band + row * EPF + 8 * c);
        const f32x4 v1 = *reinterpret_cast<const f32x4*>(band + row * EPF + 8 * c + 4);
        const int m = m0 + 32 * (wm * WM + a) + row, n = n0 + 32 * wn * WN + 8 * c;
        const bf16x8 r = *reinterpret_cast<const bf16x8*>(ep.aux + (int64_t)m * ep.ld_aux + n);
        bf16x8 w;
#pragma unroll
        for (int e = 0; e < 4; e++) w[e] = (bf16)(v0[e] + (float)r[e]), w[4 + e] = (bf16)(v1[e] + (float)r[4 + e]);
        store_out16(C + (int64_t)m * ldc + n, w);
      }
    }
    return;
  }
  if constexpr (EPI == EPI_SWIGLU_FWD) {
    constexpr int EP = 32 * WN + 8, EPH = 16 * WN + 8;
    bf16* band = reinterpret_cast<bf16*>(smem_raw) + wave * 32 * EP;
    const int j0 = n0 / 2;   // first j of the tile
#pragma unroll
    for (int a = 0; a < WM; a++) {
    LOAD_ROW(a);
      bf16x4 gu[WN][4];
#pragma unroll
      for (int b = 0; b < WN; b++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
#pragma unroll
          for (int e = 0; e < 4; e++) gu[b][q][e] = (bf16)ACC(a, b)[4 * q + e];
          *reinterpret_cast<bf16x4*>(band + i * EP + 32 * b + 8 * q + 4 * g) = gu[b][q];
        }
      constexpr int CPR = 32 * WN / 8, RPP = 64 / CPR;
#pragma unroll
      for (int pass = 0; pass < 32 / RPP; pass++) {
        const int row = pass * RPP + lane / CPR, c = lane % CPR;
        const bf16x8 w = *reinterpret_cast<const bf16x8*>(band + row * EP + 8 * c);
        const int m = m0 + 32 * (wm * WM + a) + row, blk = wn * WN + c / 4;   // 32-column block of the tile
        const int col = (blk & 1) * ep.I + j0 + 32 * (blk >> 1) + 8 * (c % 4);
        store_out16(C + (int64_t)m * ldc + col, w);
      }
      // h from the rounded values; blocks 2 p (gate) and 2 p + 1 (up) of this wavefront pair up
#pragma unroll
      for (int pr = 0; pr < WN / 2; pr++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          bf16x4 hv;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float a1 = (float)gu[2 * pr][q][e], a3 = (float)gu[2 * pr + 1][q][e];
            hv[e] = (bf16)(a1 / (1.f + __expf(-a1)) * a3);
          }
          *reinterpret_cast<bf16x4*>(band + i * EPH + 32 * pr + 8 * q + 4 * g) = hv;
        }
      constexpr int CPRH = 16 * WN / 8, RPPH = 64 / CPRH;
#pragma unroll
      for (int pass = 0; pass < 32 / RPPH; pass++) {
        const int row = pass * RPPH + lane / CPRH, c = lane % CPRH;
        const bf16x8 w = *reinterpret_cast<const bf16x8*>(band + row * EPH + 8 * c);
        const int m = m0 + 32 * (wm * WM + a) + row;
        const int col = j0 + 32 * (wn * (WN / 2) + c / 4) + 8 * (c % 4);
        store_out16(ep.out2 + (int64_t)m * ep.ld_out2 + col, w);
      }
    }
    return;
  }
  if constexpr (EPI == EPI_ROPE) {
    constexpr int EP = 32 * WN + 8;
    bf16* band = reinterpret_cast<bf16*>(smem_raw) + wave * 32 * EP;
    const bool rotate = n0 + 32 * wn * WN < ep.I;   // this wavefront's head is a query or key head
#pragma unroll
    for (int a = 0; a < WM; a++) {
    LOAD_ROW(a);
      const int mrow = m0 + 32 * (wm * WM + a) + i;   // the token this lane holds
#pragma unroll
      for (int bb = 0; bb < 2; bb++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          bf16x4 w1, w2;
          if (rotate) {
            // (cos, sin) of frequencies 32 bb + 8 q + 4 g + (0..3): 16 bytes of the token's table row
            const bf16x8 cs = *reinterpret_cast<const bf16x8*>(ep.aux + (int64_t)mrow * ep.ld_aux + 2 * (32 * bb + 8 * q + 4 * g));
#pragma unroll
            for (int e = 0; e < 4; e++) {
              const float c = (float)cs[2 * e], sn = (float)cs[2 * e + 1];
              const float x1 = ACC(a, bb)[4 * q + e], x2 = ACC(a, bb + 2)[4 * q + e];
              w1[e] = (bf16)(x1 * c - x2 * sn);
              w2[e] = (bf16)(x2 * c + x1 * sn);
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++) w1[e] = (bf16)ACC(a, bb)[4 * q + e], w2[e] = (bf16)ACC(a, bb + 2)[4 * q + e];
          }
          *reinterpret_cast<bf16x4*>(band + i * EP + 32 * bb + 8 * q + 4 * g) = w1;
          *reinterpret_cast<bf16x4*>(band + i * EP + 32 * (bb + 2) + 8 * q + 4 * g) = w2;
        }
      constexpr int CPR = 32 * WN / 8, RPP = 64 / CPR;
#pragma unroll
      for (int pass = 0; pass < 32 / RPP; pass++) {
        const int row = pass * RPP + lane / CPR, c = lane % CPR;
        const bf16x8 w = *reinterpret_cast<const bf16x8*>(band + row * EP + 8 * c);
        const int m = m0 + 32 * (wm * WM + a) + row;
        store_out16(C + (int64_t)m * ldc + n0 + 32 * wn * WN + 8 * c, w);
      }
    }
    return;
  }
  if constexpr (EPI == EPI_SWIGLU_BWD) {
    constexpr int EP = 32 * WN + 8;
    bf16* band = reinterpret_cast<bf16*>(smem_raw) + wave * 32 * EP;
#pragma unroll
    for (int a = 0; a < WM; a++) {
    LOAD_ROW(a);
#pragma unroll
      for (int b = 0; b < WN; b++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          bf16x4 w;
#pragma unroll
          for (int e = 0; e < 4; e++) w[e] = (bf16)ACC(a, b)[4 * q + e];
          *reinterpret_cast<bf16x4*>(band + i * EP + 32 * b + 8 * q + 4 * g) = w;
        }
      constexpr int CPR = 32 * WN / 8, RPP = 64 / CPR;
#pragma unroll
      for (int pass = 0; pass < 32 / RPP; pass++) {
        const int row = pass * RPP + lane / CPR, c = lane % CPR;
        const bf16x8 dh = *reinterpret_cast<const bf16x8*>(band + row * EP + 8 * c);
        const int m = m0 + 32 * (wm * WM + a) + row, j = n0 + 32 * wn * WN + 8 * c;
        const bf16x8 gt = *reinterpret_cast<const bf16x8*>(ep.aux + (int64_t)m * ep.ld_aux + j);
        const bf16x8 up = *reinterpret_cast<const bf16x8*>(ep.aux + (int64_t)m * ep.ld_aux + ep.I + j);
        bf16x8 d1, d3;
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float a1 = (float)gt[e], a3 = (float)up[e], gg = (float)dh[e];
          const float sig = 1.f / (1.f + __expf(-a1));
          d1[e] = (bf16)(gg * a3 * sig * (1.f + a1 * (1.f - sig)));
          d3[e] = (bf16)(gg * a1 * sig);
        }
        store_out16(C + (int64_t)m * ldc + j, d1);
        store_out16(C + (int64_t)m * ldc + ep.I + j, d3);
      }
    }
    return;
  }
  if (!accumulate) {
    constexpr int EP = 32 * WN + 8;                                     // band pitch in elements
    bf16* band = reinterpret_cast<bf16*>(smem_raw) + wave * 32 * EP;   // 32 rows x (32 * WN) columns per wavefront
    static_assert(4 * 32 * EP <= 2 * (TA::ELEMS + TB::ELEMS), "the bands fit in the operand buffers");
#pragma unroll
    for (int a = 0; a < WM; a++) {
    LOAD_ROW(a);
#pragma unroll
      for (int b = 0; b < WN; b++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const int nl = 32 * b + 8 * q + 4 * g;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = ACC(a, b)[4 * q + e];
          if (bias) {
            const bf16x4 bv = *reinterpret_cast<const bf16x4*>(bias + n0 + 32 * wn * WN + nl);
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] += (float)bv[e];
          }
          bf16x4 w;
#pragma unroll
          for (int e = 0; e < 4; e++) w[e] = (bf16)v[e];
          *reinterpret_cast<bf16x4*>(band + i * EP + nl) = w;
        }
      // the band is private to the wavefront and LDS operations of a wavefront complete in order
      constexpr int CPR = 32 * WN / 8, RPP = 64 / CPR;                  // 16-byte chunks per row, rows per pass
#pragma unroll
      for (int pass = 0; pass < 32 / RPP; pass++) {
        const int row = pass * RPP + lane / CPR, c = lane % CPR;
        const bf16x8 w = *reinterpret_cast<const bf16x8*>(band + row * EP + 8 * c);
        const int m = m0 + 32 * (wm * WM + a) + row;
        store_out16(C + (int64_t)m * ldc + n0 + 32 * wn * WN + 8 * c, w);
      }
    }
    return;
  }
#pragma unroll
  for (int a = 0; a < WM; a++) {
    LOAD_ROW(a);
    const int m = m0 + 32 * (wm * WM + a) + i;
#pragma unroll
    for (int b = 0; b < WN; b++) {
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int n = n0 + 32 * (wn * WN + b) + 8 * q + 4 * g;
        bf16* dst = C + (int64_t)m * ldc + n;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = ACC(a, b)[4 * q + e];
        if (bias) {
          const bf16x4 bv = *reinterpret_cast<const bf16x4*>(bias + n);
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] += (float)bv[e];
        }
        if (accumulate) {
          const bf16x4 old = *reinterpret_cast<const bf16x4*>(dst);
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] += (float)old[e];
        }
        bf16x4 w;
#pragma unroll
        for (int e = 0; e < 4; e++) w[e] = (bf16)v[e];
        *reinterpret_cast<bf16x4*>(dst) = w;
      }
    }
  }
}

#undef ACC
#undef LOAD_ROW

template <int WM, int WN, bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(const bf16* __restrict__ A, const bf16* __restrict__ B,
                                                        bf16* __restrict__ C, const bf16* __restrict__ bias, int M,
                                                        int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
                                                        int accumulate, int tiles_m, int tiles_n) {
  constexpr int TM = 64 * WM, TN = 64 * WN;  // block tile
  typedef OperandTile<TM, A_KC> TA;
  typedef OperandTile<TN, B_KC> TB;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* As = reinterpret_cast<bf16*>(smem_raw);  // [2][TA::ELEMS]
  bf16* Bs = As + 2 * TA::ELEMS;                 // [2][TB::ELEMS]

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 5, i = lane & 31;
  const int wm = wave >> 1, wn = wave & 1;

  // Block -> tile.  Consecutive workgroup ids go round-robin over the 8 XCDs, each
  // with its own L2: give every XCD a contiguous range of tiles, and inside the
  // range walk down M in groups so that neighbours share the B panel.
  int pid = blockIdx.x;
  const int nblk = tiles_m * tiles_n;
  if (nblk % 8 == 0) pid = (pid % 8) * (nblk / 8) + pid / 8;
  constexpr int GROUP = 8;
  const int per_group = GROUP * tiles_n;
  const int gid = pid / per_group, first_m = gid * GROUP;
  const int gsz = min(tiles_m - first_m, GROUP);
  const int tm = first_m + (pid % per_group) % gsz, tn = (pid % per_group) / gsz;
  const int m0 = tm * TM, n0 = tn * TN;

  f32x16 acc[WM][WN];
#pragma unroll
  for (int a = 0; a < WM; a++)
#pragma unroll
    for (int b = 0; b < WN; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

  TA ta;
  TB tb;
  const int nk = (K + BK - 1) / BK;
  ta.gload(A, lda, m0, 0, M, K, tid);
  tb.gload(B, ldb, n0, 0, N, K, tid);
  ta.sstore(As, tid);
  tb.sstore(Bs, tid);
  __syncthreads();

  for (int kt = 0; kt < nk; kt++) {
    const int buf = kt & 1;
    if (kt + 1 < nk) {
      ta.gload(A, lda, m0, (kt + 1) * BK, M, K, tid);
      tb.gload(B, ldb, n0, (kt + 1) * BK, N, K, tid);
    }
    const bf16* Ab = As + buf * TA::ELEMS;
    const bf16* Bb = Bs + buf * TB::ELEMS;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      bf16x8 af[WM], bfr[WN];
#pragma unroll
      for (int a = 0; a < WM; a++) af[a] = TA::frag(Ab, 32 * (wm * WM + a), ks, g, i);
#pragma unroll
      for (int b = 0; b < WN; b++) bfr[b] = TB::frag(Bb, 32 * (wn * WN + b), ks, g, i);
#pragma unroll
      for (int a = 0; a < WM; a++)
#pragma unroll
        for (int b = 0; b < WN; b++) acc[a][b] = mfma32(bfr[b], af[a], acc[a][b]);  // rows = n, cols = m
    }
    if (kt + 1 < nk) {
      ta.sstore(As + (buf ^ 1) * TA::ELEMS, tid);
      tb.sstore(Bs + (buf ^ 1) * TB::ELEMS, tid);
    }
    __syncthreads();
  }

  // epilogue: lane (g, i) holds column m = i, rows n = 8*(r/4) + 4g + r%4
#pragma unroll
  for (int a = 0; a < WM; a++) {
    const int m = m0 + 32 * (wm * WM + a) + i;
    if (m >= M) continue;
#pragma unroll
    for (int b = 0; b < WN; b++) {
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int n = n0 + 32 * (wn * WN + b) + 8 * q + 4 * g;
        if (n >= N) continue;  // N % 8 == 0: a quad is all in or all out
        bf16* dst = C + (int64_t)m * ldc + n;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = acc[a][b][4 * q + e];
        if (bias) {
          const bf16x4 bv = *reinterpret_cast<const bf16x4*>(bias + n);
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] += (float)bv[e];
        }
        if (accumulate) {
          const bf16x4 old = *reinterpret_cast<const bf16x4*>(dst);
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] += (float)old[e];
        }
        bf16x4 w;
#pragma unroll
        for (int e = 0; e < 4; e++) w[e] = (bf16)v[e];
        *reinterpret_cast<bf16x4*>(dst) = w;
      }
    }
  }
}

// C = sum over the K ranges of the fp32 partial tiles (+ bias, + C), rounded once; 4 elements per thread
__global__ __launch_bounds__(256) void gemm_splitk_sum_kernel(const float* __restrict__ part, int splits,
                                                              bf16* __restrict__ C, const bf16* __restrict__ bias, int M,
                                                              int N, int64_t ldc, int accumulate) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x, total = (int64_t)M * (N / 4);
  if (idx >= total) return;
  const int m = idx / (N / 4), n = (idx % (N / 4)) * 4;
  f32x4 v = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < splits; s++) v += *reinterpret_cast<const f32x4*>(part + ((int64_t)s * M + m) * N + n);
  if (bias) {
    const bf16x4 bv = *reinterpret_cast<const bf16x4*>(bias + n);
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] += (float)bv[e];
  }
  bf16* dst = C + (int64_t)m * ldc + n;
  if (accumulate) {
    const bf16x4 old = *reinterpret_cast<const bf16x4*>(dst);
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] += (float)old[e];
  }
  bf16x4 w;
#pragma unroll
  for (int e = 0; e < 4; e++) w[e] = (bf16)v[e];
  *reinterpret_cast<bf16x4*>(dst) = w;
}

// Number of K ranges for a product of full 256 x 256 tiles: only where the tiles alone would leave most
// of the chip idle, and every range keeps at least 8 slabs.
int splitk_plan(int M, int N, int K) {
  if (M % 256 || N % 256 || K % BK) return 1;
  const int64_t tiles = (int64_t)(M / 256) * (N / 256);
  const int nk = K / BK;
  if (tiles > 128) return 1;
  int splits = (int)(512 / tiles);
  if (splits > 8) splits = 8;
  if (splits > nk / 8) splits = nk / 8;
  return splits < 2 ? 1 : splits;
}

template <int WM, int WN, bool A_KC, bool B_KC>
int launch_bf16(const bf16* A, const bf16* B, bf16* C, const bf16* bias, int M, int N, int K, int64_t lda, int64_t ldb,
                int64_t ldc, int accumulate, float* part, int splits, hipStream_t st) {
  constexpr int TM = 64 * WM, TN = 64 * WN;
  constexpr size_t smem = 2 * sizeof(bf16) * (OperandTile<TM, A_KC>::ELEMS + OperandTile<TN, B_KC>::ELEMS);
  auto kern = &gemm_bf16_kernel<WM, WN, A_KC, B_KC>;
  auto fast = &gemm_bf16_fast_kernel<WM, WN, A_KC, B_KC, false>;
  auto fastk = &gemm_bf16_fast_kernel<WM, WN, A_KC, B_KC, true>;
  for (const void* f : {reinterpret_cast<const void*>(kern), reinterpret_cast<const void*>(fast),
                        reinterpret_cast<const void*>(fastk)})
    if (int rc = ody_allow_dynamic_lds(f, smem, "ody_gemm")) return rc;
  const int tiles_m = (M + TM - 1) / TM, tiles_n = (N + TN - 1) / TN;
  const char* name = A_KC ? (B_KC ? "gemm_bf16_nt" : "gemm_bf16_nn") : "gemm_bf16_tn";
  // per-thread offsets inside a tile are kept in 32 bits by the fast kernel, and it writes C in 16-byte pieces
  const bool interior = M % TM == 0 && N % TN == 0 && K % BK == 0 && (int64_t)TM * lda < (1ll << 31) &&
                        ody_aligned16(C) && ldc % 8 == 0 &&
                        (int64_t)TN * ldb < (1ll << 31) && (int64_t)BK * lda < (1ll << 31) &&
                        (int64_t)BK * ldb < (1ll << 31);
  if (interior && splits > 1) {
    ODY_LAUNCH(name, st, fastk, dim3(tiles_m * tiles_n, splits), dim3(256), smem, A, B, C, bias, M, N, K, lda, ldb, ldc,
               accumulate, tiles_m, tiles_n, part, GemmEpi{});
    int rc = ody_check_launch("gemm_bf16");
    if (rc) return rc;
    const int64_t n4 = (int64_t)M * (N / 4);
    ODY_LAUNCH("gemm_splitk_sum", st, gemm_splitk_sum_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, part,
               splits, C, bias, M, N, ldc, accumulate);
    return ody_check_launch("gemm_splitk_sum");
  }
  if (interior) {
    ODY_LAUNCH(name, st, fast, dim3(tiles_m * tiles_n), dim3(256), smem, A, B, C, bias, M, N, K, lda, ldb, ldc,
               accumulate, tiles_m, tiles_n, nullptr, GemmEpi{});
    return ody_check_launch("gemm_bf16");
  }
  ODY_LAUNCH(name, st, kern, dim3(tiles_m * tiles_n), dim3(256), smem, A, B, C, bias, M, N, K, lda, ldb, ldc,
             accumulate, tiles_m, tiles_n);
  return ody_check_launch("gemm_bf16");
}

template <bool A_KC, bool B_KC>
int dispatch_bf16(const bf16* A, const bf16* B, bf16* C, const bf16* bias, int M, int N, int K, int64_t lda,
                  int64_t ldb, int64_t ldc, int accumulate, void* workspace, size_t workspace_bytes, hipStream_t st) {
  // long K, few output tiles, and the caller brought the workspace: 256 x 256 tiles over ranges of K
  const int splits = splitk_plan(M, N, K);
  if (splits > 1 && workspace && workspace_bytes >= (size_t)splits * M * N * sizeof(float) && ody_aligned16(workspace) &&
      ody_aligned16(C) && ldc % 8 == 0)
    return launch_bf16<4, 4, A_KC, B_KC>(A, B, C, bias, M, N, K, lda, ldb, ldc, accumulate,
                                         static_cast<float*>(workspace), splits, st);
  // large problems: 256 x 256 tiles; otherwise 128 x 128 so that the grid still covers the chip
  const int64_t big_tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
  if (big_tiles >= 192)
    return launch_bf16<4, 4, A_KC, B_KC>(A, B, C, bias, M, N, K, lda, ldb, ldc, accumulate, nullptr, 1, st);
  return launch_bf16<2, 2, A_KC, B_KC>(A, B, C, bias, M, N, K, lda, ldb, ldc, accumulate, nullptr, 1, st);
}

// Whether a product of these sizes can take the 256 x 256 fast kernel in one pass over K (what the fused epilogues need).
bool fused_shape_ok(int M, int N, int K, int64_t lda, int64_t ldb) {
  return M % 256 == 0 && N % 256 == 0 && K % BK == 0 && 256 * lda < (1ll << 31) && 256 * ldb < (1ll << 31) &&
         BK * lda < (1ll << 31) && BK * ldb < (1ll << 31);
}

template <bool B_KC, int EPI>
int launch_fused(const char* name, const bf16* A, const bf16* B, bf16* C, int M, int N, int K, int64_t lda, int64_t ldb,
                 int64_t ldc, const GemmEpi& ep, hipStream_t st) {
  constexpr size_t smem = 2 * sizeof(bf16) * (OperandTile<256, true>::ELEMS + OperandTile<256, B_KC>::ELEMS);
  auto kern = &gemm_bf16_fast_kernel<4, 4, true, B_KC, false, EPI>;
  if (int rc = ody_allow_dynamic_lds(reinterpret_cast<const void*>(kern), smem, name)) return rc;
  const int tiles_m = M / 256, tiles_n = N / 256;
  ODY_LAUNCH(name, st, kern, dim3(tiles_m * tiles_n), dim3(256), smem, A, B, C, static_cast<const bf16*>(nullptr), M, N,
             K, lda, ldb, ldc, 0, tiles_m, tiles_n, static_cast<float*>(nullptr), ep);
  return ody_check_launch(name);
}

// One bf16 product.  A ragged M or N is cut into a main part of whole tiles, which takes the fast
// kernel, and an edge strip on the right and at the bottom for the general kernel.
int gemm_bf16(int op, const bf16* a, const bf16* b, bf16* c, const bf16* bias, int M, int N, int K, int64_t lda,
              int64_t ldb, int64_t ldc, int accumulate, void* workspace, size_t workspace_bytes, hipStream_t st) {
  const int64_t big_tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
  const int tile = big_tiles >= 192 ? 256 : 128;
  const int M0 = M / tile * tile, N0 = N / tile * tile;
  if (K % BK == 0 && M0 > 0 && N0 > 0 && (M0 < M || N0 < N)) {
    int rc = gemm_bf16(op, a, b, c, bias, M0, N0, K, lda, ldb, ldc, accumulate, workspace, workspace_bytes, st);
    if (rc) return rc;
    if (N0 < N) {   // right strip: every row, columns [N0, N)
      const bf16* b1 = (op == ODY_GEMM_NT) ? b + (int64_t)N0 * ldb : b + N0;
      rc = gemm_bf16(op, a, b1, c + N0, bias ? bias + N0 : nullptr, M, N - N0, K, lda, ldb, ldc, accumulate, nullptr, 0, st);
      if (rc) return rc;
    }
    if (M0 < M) {   // bottom strip: rows [M0, M), columns [0, N0)
      const bf16* a1 = (op == ODY_GEMM_TN) ? a + M0 : a + (int64_t)M0 * lda;
      rc = gemm_bf16(op, a1, b, c + (int64_t)M0 * ldc, bias, M - M0, N0, K, lda, ldb, ldc, accumulate, nullptr, 0, st);
    }
    return rc;
  }
  if (op == ODY_GEMM_NT)
    return dispatch_bf16<true, true>(a, b, c, bias, M, N, K, lda, ldb, ldc, accumulate, workspace, workspace_bytes, st);
  if (op == ODY_GEMM_NN)
    return dispatch_bf16<true, false>(a, b, c, bias, M, N, K, lda, ldb, ldc, accumulate, workspace, workspace_bytes, st);
  return dispatch_bf16<false, false>(a, b, c, bias, M, N, K, lda, ldb, ldc, accumulate, workspace, workspace_bytes, st);
}

// ------------------------------------------------------------------ fp32 MFMA
constexpr int FK = 32;  // K-slab of the fp32 kernel

__device__ __forceinline__ f32x16 mfma_f32(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// One operand slab (BT rows x FK of K) on its way from global memory to LDS and out again as
// MFMA fragments.  KC = true: memory is (rows, K) row-major, LDS [BT][FK + 4], a fragment is one
// 16-byte read.  KC = false: memory is (K, rows) row-major, LDS [FK][BT + 8], a fragment is four
// 4-byte reads.  Either way k-step 4 j + t of lane half g multiplies K index 8 j + 4 g + t, so
// both operands of a product agree, and both pitches keep the reads conflict-free.
template <int BT, bool KC>
struct F32Tile {
  static constexpr int PITCH = KC ? FK + 4 : BT + 8;
  static constexpr int ELEMS = (KC ? BT : FK) * PITCH;
  static constexpr int CHUNKS = BT * FK / 4 / 256;  // 16-byte pieces per thread
  f32x4 r[CHUNKS];

  static __device__ __forceinline__ void coord(int c, int& rr, int& kk) {
    if (KC) { rr = c / (FK / 4); kk = (c % (FK / 4)) * 4; }
    else { kk = c / (BT / 4); rr = (c % (BT / 4)) * 4; }
  }
  // row0: first row (M or N index) of the tile; k0: first K index; out-of-range elements read as 0
  template <bool VEC>
  __device__ __forceinline__ void gload(const float* base, int64_t ld, int row0, int k0, int nrows, int K, int tid) {
#pragma unroll
    for (int j = 0; j < CHUNKS; j++) {
      int rr, kk;
      coord(tid + 256 * j, rr, kk);
      const int row = row0 + rr, k = k0 + kk;
      const float* src = KC ? base + (int64_t)row * ld + k : base + (int64_t)k * ld + row;
      if (VEC) {
        r[j] = (row < nrows && k < K) ? *reinterpret_cast<const f32x4*>(src) : f32x4{0.f, 0.f, 0.f, 0.f};
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const bool ok = KC ? (row < nrows && k + e < K) : (row + e < nrows && k < K);
          r[j][e] = ok ? src[e] : 0.f;
        }
      }
    }
  }
  __device__ __forceinline__ void put(float* lds, int tid) const {
#pragma unroll
    for (int j = 0; j < CHUNKS; j++) {
      int rr, kk;
      coord(tid + 256 * j, rr, kk);
      *reinterpret_cast<f32x4*>(lds + (KC ? rr * PITCH + kk : kk * PITCH + rr)) = r[j];
    }
  }
  // k-steps 4 j .. 4 j + 3 of row r0 + i
  static __device__ __forceinline__ f32x4 frag(const float* lds, int r0, int i, int g, int j) {
    if (KC) return *reinterpret_cast<const f32x4*>(lds + (r0 + i) * PITCH + 8 * j + 4 * g);
    f32x4 v;
#pragma unroll
    for (int t = 0; t < 4; t++) v[t] = lds[(8 * j + 4 * g + t) * PITCH + r0 + i];
    return v;
  }
};

// v_mfma_f32_32x32x2_f32, 4 wavefronts in a 2 x 2 arrangement, each owning WT x WT result tiles
// of 32 x 32 (a 64 x 64 or 128 x 128 workgroup tile).  One LDS slab; the next one is fetched into
// registers while the current one is multiplied.  The product is computed as C^T = op(B)^T op(A)^T,
// so a lane holds 4 consecutive N per register quad and writes 16-byte pieces of C rows.
// VEC = false (unaligned pointers or extents that are not multiples of 4) moves single floats.
template <int WT, bool A_KC, bool B_KC, bool VEC>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                       float* __restrict__ C, const float* __restrict__ bias, int M,
                                                       int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
                                                       int accumulate, int ntn) {
  constexpr int BT = 64 * WT;
  constexpr int NCH = (WT == 1) ? 2 : 1;  // never a single chain of dependent MFMAs
  using TA = F32Tile<BT, A_KC>;
  using TB = F32Tile<BT, B_KC>;
  __shared__ __attribute__((aligned(16))) float As[TA::ELEMS];
  __shared__ __attribute__((aligned(16))) float Bs[TB::ELEMS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i = lane & 31, g = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = (blockIdx.x / ntn) * BT, n0 = (blockIdx.x % ntn) * BT;

  f32x16 acc[WT][WT][NCH];
#pragma unroll
  for (int a = 0; a < WT; a++)
#pragma unroll
    for (int b = 0; b < WT; b++)
#pragma unroll
      for (int c = 0; c < NCH; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[a][b][c][r] = 0.f;

  TA ta;
  TB tb;
  ta.template gload<VEC>(A, lda, m0, 0, M, K, tid);
  tb.template gload<VEC>(B, ldb, n0, 0, N, K, tid);
  for (int k0 = 0; k0 < K; k0 += FK) {
    __syncthreads();
    ta.put(As, tid);
    tb.put(Bs, tid);
    __syncthreads();
    if (k0 + FK < K) {
      ta.template gload<VEC>(A, lda, m0, k0 + FK, M, K, tid);
      tb.template gload<VEC>(B, ldb, n0, k0 + FK, N, K, tid);
    }
#pragma unroll
    for (int j = 0; j < FK / 8; j++) {
      f32x4 af[WT], bf[WT];
#pragma unroll
      for (int a = 0; a < WT; a++) af[a] = TA::frag(As, 32 * (wm * WT + a), i, g, j);
#pragma unroll
      for (int b = 0; b < WT; b++) bf[b] = TB::frag(Bs, 32 * (wn * WT + b), i, g, j);
#pragma unroll
      for (int t = 0; t < 4; t++)
#pragma unroll
        for (int a = 0; a < WT; a++)
#pragma unroll
          for (int b = 0; b < WT; b++)
            acc[a][b][t % NCH] = mfma_f32(bf[b][t], af[a][t], acc[a][b][t % NCH]);
    }
  }

  // register r of lane (i, g) of tile (a, b): row m = 32 (wm WT + a) + i, column n = 32 (wn WT + b) + 8 (r / 4) + 4 g + r % 4
#pragma unroll
  for (int a = 0; a < WT; a++) {
    const int m = m0 + 32 * (wm * WT + a) + i;
    if (m >= M) continue;
#pragma unroll
    for (int b = 0; b < WT; b++) {
      f32x16 v = acc[a][b][0];
      if (NCH == 2) v += acc[a][b][NCH - 1];
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int n = n0 + 32 * (wn * WT + b) + 8 * q + 4 * g;
        float* dst = C + (int64_t)m * ldc + n;
        if (VEC && n + 3 < N) {
          f32x4 o{v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
          if (bias) o += *reinterpret_cast<const f32x4*>(bias + n);
          if (accumulate) o += *reinterpret_cast<const f32x4*>(dst);
          *reinterpret_cast<f32x4*>(dst) = o;
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++) {
            if (n + e >= N) continue;
            float o = v[4 * q + e];
            if (bias) o += bias[n + e];
            if (accumulate) o += dst[e];
            dst[e] = o;
          }
        }
      }
    }
  }
}

template <int WT, bool A_KC, bool B_KC>
int launch_f32(const float* a, const float* b, float* c, const float* bias, int M, int N, int K, int64_t lda,
               int64_t ldb, int64_t ldc, int accumulate, bool vec, hipStream_t st) {
  constexpr int BT = 64 * WT;
  const int64_t ntm = (M + BT - 1) / BT, ntn = (N + BT - 1) / BT;
  ODY_REQUIRE(ntm * ntn < ((int64_t)1 << 31), ODY_ERR_BAD_SHAPE, "ody_gemm: M=%d N=%d too large for one launch", M, N);
  const dim3 grid((unsigned)(ntm * ntn)), blk(256);
  if (vec)
    ODY_LAUNCH("gemm_f32", st, (gemm_f32_kernel<WT, A_KC, B_KC, true>), grid, blk, 0, a, b, c, bias, M, N, K, lda,
               ldb, ldc, accumulate, (int)ntn);
  else
    ODY_LAUNCH("gemm_f32", st, (gemm_f32_kernel<WT, A_KC, B_KC, false>), grid, blk, 0, a, b, c, bias, M, N, K, lda,
               ldb, ldc, accumulate, (int)ntn);
  return ody_check_launch("gemm_f32");
}

template <bool A_KC, bool B_KC>
int dispatch_f32(const float* a, const float* b, float* c, const float* bias, int M, int N, int K, int64_t lda,
                 int64_t ldb, int64_t ldc, int accumulate, hipStream_t st) {
  const bool vec = ody_aligned16(a) && ody_aligned16(b) && ody_aligned16(c) && (!bias || ody_aligned16(bias)) &&
                   lda % 4 == 0 && ldb % 4 == 0 && ldc % 4 == 0 && M % 4 == 0 && N % 4 == 0 && K % 4 == 0;
  // 128 x 128 tiles once they fill the chip twice over, 64 x 64 tiles below that
  const int64_t big = (int64_t)((M + 127) / 128) * ((N + 127) / 128);
  if (big >= 512) return launch_f32<2, A_KC, B_KC>(a, b, c, bias, M, N, K, lda, ldb, ldc, accumulate, vec, st);
  return launch_f32<1, A_KC, B_KC>(a, b, c, bias, M, N, K, lda, ldb, ldc, accumulate, vec, st);
}

int gemm_f32(int op, const float* a, const float* b, float* c, const float* bias, int M, int N, int K, int64_t lda,
             int64_t ldb, int64_t ldc, int accumulate, hipStream_t st) {
  if (op == ODY_GEMM_NT) return dispatch_f32<true, true>(a, b, c, bias, M, N, K, lda, ldb, ldc, accumulate, st);
  if (op == ODY_GEMM_NN) return dispatch_f32<true, false>(a, b, c, bias, M, N, K, lda, ldb, ldc, accumulate, st);
  return dispatch_f32<false, false>(a, b, c, bias, M, N, K, lda, ldb, ldc, accumulate, st);
}

}  // namespace

extern "C" size_t ody_gemm_workspace_bytes(int op, int M, int N, int K, int dtype) {
  (void)op;
  if (dtype != ODY_BF16 || M <= 0 || N <= 0 || K <= 0) return 0;
  const int splits = splitk_plan(M, N, K);
  return splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
}

extern "C" int ody_gemm(int op, const void* A, const void* B, void* C, const void* bias, int M, int N, int K,
                        int64_t lda, int64_t ldb, int64_t ldc, int accumulate, int dtype, void* workspace,
                        size_t workspace_bytes, void* stream) {
  ODY_REQUIRE(A && B && C, ODY_ERR_NULL, "ody_gemm: NULL pointer");
  ODY_REQUIRE(M > 0 && N > 0 && K > 0, ODY_ERR_BAD_SHAPE, "ody_gemm: M=%d N=%d K=%d", M, N, K);
  ODY_REQUIRE(op == ODY_GEMM_NT || op == ODY_GEMM_NN || op == ODY_GEMM_TN, ODY_ERR_UNSUPPORTED, "ody_gemm: op %d", op);
  const int a_cols = (op == ODY_GEMM_TN) ? M : K, b_cols = (op == ODY_GEMM_NT) ? K : N;
  ODY_REQUIRE(lda >= a_cols && ldb >= b_cols && ldc >= N, ODY_ERR_BAD_SHAPE,
              "ody_gemm: leading dimension smaller than the row length (lda=%lld ldb=%lld ldc=%lld)", (long long)lda,
              (long long)ldb, (long long)ldc);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == ODY_F32)
    return gemm_f32(op, (const float*)A, (const float*)B, (float*)C, (const float*)bias, M, N, K, lda, ldb, ldc,
                    accumulate, st);
  ODY_REQUIRE(dtype == ODY_BF16, ODY_ERR_UNSUPPORTED, "ody_gemm: dtype %d unknown", dtype);
  // 16-byte vectors along the contiguous direction of every matrix
  ODY_REQUIRE(ody_aligned16(A) && ody_aligned16(B) && ((reinterpret_cast<uintptr_t>(C) & 7u) == 0) &&
                  (!bias || (reinterpret_cast<uintptr_t>(bias) & 7u) == 0),
              ODY_ERR_MISALIGNED, "ody_gemm: A and B must be 16-byte aligned, C and bias 8-byte aligned");
  ODY_REQUIRE(lda % 8 == 0 && ldb % 8 == 0 && ldc % 4 == 0, ODY_ERR_MISALIGNED,
              "ody_gemm: lda and ldb must be multiples of 8, ldc of 4");
  ODY_REQUIRE(N % 8 == 0 && a_cols % 8 == 0 && b_cols % 8 == 0, ODY_ERR_UNSUPPORTED,
              "ody_gemm: bf16 path needs N and the contiguous extents of A and B to be multiples of 8 "
              "(M=%d N=%d K=%d op=%d)", M, N, K, op);
  return gemm_bf16(op, (const bf16*)A, (const bf16*)B, (bf16*)C, (const bf16*)bias, M, N, K, lda, ldb, ldc, accumulate,
                   workspace, workspace_bytes, st);
}

// ---------------------------------------------------------------------------
// Linears with the neighbouring elementwise operation in their epilogue
// ---------------------------------------------------------------------------
namespace {
int check_lin(const char* who, const void* a, const void* b, const void* c, int M, int N, int K, int dtype) {
  ODY_REQUIRE(a && b && c, ODY_ERR_NULL, "%s: NULL pointer", who);
  ODY_REQUIRE(M > 0 && N > 0 && K > 0, ODY_ERR_BAD_SHAPE, "%s: M=%d N=%d K=%d", who, M, N, K);
  ODY_REQUIRE(dtype == ODY_BF16 || dtype == ODY_F32, ODY_ERR_UNSUPPORTED, "%s: dtype %d unknown", who, dtype);
  return ODY_OK;
}
bool vec16(const void* p, int64_t ld) { return ody_aligned16(p) && ld % 8 == 0; }
}  // namespace

extern "C" int ody_linear_rope(const void* x, const void* w, const void* table, void* y, int M, int N, int K, int n_rot,
                              int D, int64_t ldx, int64_t ldw, int64_t ld_table, int64_t ldy, int dtype, void* stream) {
  int rc = check_lin("ody_linear_rope", x, w, y, M, N, K, dtype);
  if (rc) return rc;
  ODY_REQUIRE(table != nullptr, ODY_ERR_NULL, "ody_linear_rope: table is NULL");
  ODY_REQUIRE(dtype == ODY_BF16 && D == 128, ODY_ERR_UNSUPPORTED, "ody_linear_rope: bf16 and head_dim 128 only");
  ODY_REQUIRE(n_rot >= 0 && N % D == 0 && n_rot <= N / D, ODY_ERR_BAD_SHAPE, "ody_linear_rope: N=%d n_rot=%d D=%d", N, n_rot, D);
  ODY_REQUIRE(ldx >= K && ldw >= K && ldy >= N, ODY_ERR_BAD_SHAPE, "ody_linear_rope: leading dimension smaller than the row length");
  ODY_REQUIRE(ld_table == D, ODY_ERR_BAD_SHAPE, "ody_linear_rope: the table's rows are D = %d elements apart, got %lld", D,
              (long long)ld_table);
  ODY_REQUIRE(vec16(table, ld_table) && vec16(y, ldy), ODY_ERR_MISALIGNED,
              "ody_linear_rope: table and y need 16-byte aligned rows");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (fused_shape_ok(M, N, K, ldx, ldw) && vec16(x, ldx) && vec16(w, ldw)) {
    GemmEpi ep{static_cast<const bf16*>(table), nullptr, ld_table, 0, n_rot * D};
    return launch_fused<true, EPI_ROPE>("gemm_bf16_nt_rope", static_cast<const bf16*>(x), static_cast<const bf16*>(w),
                                        static_cast<bf16*>(y), M, N, K, ldx, ldw, ldy, ep, st);
  }
  // other shapes: the plain product, then the rotation in place (one more rounding of the rotated columns)
  rc = ody_gemm(ODY_GEMM_NT, x, w, y, nullptr, M, N, K, ldx, ldw, ldy, 0, dtype, nullptr, 0, stream);
  if (rc) return rc;
  return ody_launch_rope_from_table(y, table, M, n_rot, D, ldy, D, 0, st);
}

extern "C" int ody_linear_residual(const void* x, const void* w, const void* residual, void* y, int M, int N, int K,
                                   int64_t ldx, int64_t ldw, int64_t ld_res, int64_t ldy, int dtype, void* stream) {
  int rc = check_lin("ody_linear_residual", x, w, y, M, N, K, dtype);
  if (rc) return rc;
  ODY_REQUIRE(residual != nullptr, ODY_ERR_NULL, "ody_linear_residual: residual is NULL");
  ODY_REQUIRE(ldx >= K && ldw >= K && ld_res >= N && ldy >= N, ODY_ERR_BAD_SHAPE,
              "ody_linear_residual: leading dimension smaller than the row length");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == ODY_BF16 && fused_shape_ok(M, N, K, ldx, ldw) && vec16(x, ldx) && vec16(w, ldw) && vec16(residual, ld_res) &&
      vec16(y, ldy) && (int64_t)((M + 255) / 256) * ((N + 255) / 256) >= 128) {
    GemmEpi ep{static_cast<const bf16*>(residual), nullptr, ld_res, 0, 0};
    return launch_fused<true, EPI_RESIDUAL>("gemm_bf16_nt_residual", static_cast<const bf16*>(x), static_cast<const bf16*>(w),
                                            static_cast<bf16*>(y), M, N, K, ldx, ldw, ldy, ep, st);
  }
  // any other shape or type: y = residual, then y += x W^T (added in fp32 before the one rounding, as above)
  if (y != residual) {
    const size_t es = dtype == ODY_BF16 ? 2 : 4;
    hipError_t e = hipMemcpy2DAsync(y, (size_t)ldy * es, residual, (size_t)ld_res * es, (size_t)N * es, (size_t)M,
                                    hipMemcpyDeviceToDevice, st);
    ODY_REQUIRE(e == hipSuccess, ODY_ERR_LAUNCH, "ody_linear_residual: copy of the residual failed: %s", hipGetErrorString(e));
  }
  return ody_gemm(ODY_GEMM_NT, x, w, y, nullptr, M, N, K, ldx, ldw, ldy, 1, dtype, nullptr, 0, stream);
}

extern "C" int ody_swiglu_fwd(const void* gate_up, void* h, int T, int I, int64_t ld_gu, int64_t ld_h, int dtype,
                              void* stream);
extern "C" int ody_swiglu_bwd(const void* gate_up, const void* dh, void* d_gate_up, int T, int I, int64_t ld_gu,
                              int64_t ld_dh, int64_t ld_dgu, int dtype, void* stream);

extern "C" int ody_linear_swiglu(const void* x, const void* w_gate_up, void* gate_up, void* h, int T, int I, int K,
                                 int64_t ldx, int64_t ldw, int64_t ld_gu, int64_t ld_h, int dtype, void* stream) {
  int rc = check_lin("ody_linear_swiglu", x, w_gate_up, gate_up, T, I, K, dtype);
  if (rc) return rc;
  ODY_REQUIRE(h != nullptr, ODY_ERR_NULL, "ody_linear_swiglu: h is NULL");
  ODY_REQUIRE(ldx >= K && ldw >= K && ld_gu >= 2 * (int64_t)I && ld_h >= I, ODY_ERR_BAD_SHAPE,
              "ody_linear_swiglu: leading dimension smaller than the row length");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == ODY_BF16 && I % 128 == 0 && fused_shape_ok(T, 2 * I, K, ldx, ldw) && (int64_t)I * ldw < (1ll << 40) &&
      vec16(x, ldx) && vec16(w_gate_up, ldw) && vec16(gate_up, ld_gu) && vec16(h, ld_h)) {
    GemmEpi ep{nullptr, static_cast<bf16*>(h), 0, ld_h, I};
    return launch_fused<true, EPI_SWIGLU_FWD>("gemm_bf16_nt_swiglu", static_cast<const bf16*>(x),
                                              static_cast<const bf16*>(w_gate_up), static_cast<bf16*>(gate_up), T, 2 * I, K,
                                              ldx, ldw, ld_gu, ep, st);
  }
  rc = ody_gemm(ODY_GEMM_NT, x, w_gate_up, gate_up, nullptr, T, 2 * I, K, ldx, ldw, ld_gu, 0, dtype, nullptr, 0, stream);
  if (rc) return rc;
  return ody_swiglu_fwd(gate_up, h, T, I, ld_gu, ld_h, dtype, stream);
}

extern "C" size_t ody_linear_dgrad_swiglu_workspace_bytes(int T, int I, int K, int dtype) {
  if (T <= 0 || I <= 0 || K <= 0) return 0;
  if (dtype == ODY_BF16 && T % 256 == 0 && I % 256 == 0 && K % BK == 0) return 0;
  return (((size_t)T * I * (dtype == ODY_BF16 ? 2 : 4)) + 255) & ~(size_t)255;
}

extern "C" int ody_linear_dgrad_swiglu(const void* dy, const void* w_down, const void* gate_up, void* d_gate_up, int T,
                                       int I, int K, int64_t ld_dy, int64_t ldw, int64_t ld_gu, int64_t ld_dgu, int dtype,
                                       void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_lin("ody_linear_dgrad_swiglu", dy, w_down, d_gate_up, T, I, K, dtype);
  if (rc) return rc;
  ODY_REQUIRE(gate_up != nullptr, ODY_ERR_NULL, "ody_linear_dgrad_swiglu: gate_up is NULL");
  ODY_REQUIRE(ld_dy >= K && ldw >= I && ld_gu >= 2 * (int64_t)I && ld_dgu >= 2 * (int64_t)I, ODY_ERR_BAD_SHAPE,
              "ody_linear_dgrad_swiglu: leading dimension smaller than the row length");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == ODY_BF16 && fused_shape_ok(T, I, K, ld_dy, ldw) && vec16(dy, ld_dy) && vec16(w_down, ldw) &&
      vec16(gate_up, ld_gu) && vec16(d_gate_up, ld_dgu)) {
    GemmEpi ep{static_cast<const bf16*>(gate_up), nullptr, ld_gu, 0, I};
    return launch_fused<false, EPI_SWIGLU_BWD>("gemm_bf16_nn_swiglu_bwd", static_cast<const bf16*>(dy),
                                               static_cast<const bf16*>(w_down), static_cast<bf16*>(d_gate_up), T, I, K,
                                               ld_dy, ldw, ld_dgu, ep, st);
  }
  const size_t need = (size_t)T * I * (dtype == ODY_BF16 ? 2 : 4);
  ODY_REQUIRE(workspace != nullptr && workspace_bytes >= need && ody_aligned16(workspace), ODY_ERR_WORKSPACE,
              "ody_linear_dgrad_swiglu: this shape runs as two kernels and needs a 16-byte aligned workspace of %zu bytes "
              "for dh (got %zu)", need, workspace ? workspace_bytes : (size_t)0);
  rc = ody_gemm(ODY_GEMM_NN, dy, w_down, workspace, nullptr, T, I, K, ld_dy, ldw, I, 0, dtype, nullptr, 0, stream);
  if (rc) return rc;
  return ody_swiglu_bwd(gate_up, workspace, d_gate_up, T, I, ld_gu, I, ld_dgu, dtype, stream);
}
