// LDS tiles of the head_dim-128 attention kernels: 64 rows x 128 bf16, filled by direct
// global->LDS loads and read with 16-byte reads, without bank conflicts and with purely
// additive addressing.
//
// A direct load (global_load_lds_dwordx4) makes the 64 lanes of a wavefront write
// 64 consecutive 16-byte slots of LDS, each lane fetching from its own global
// address.  One such load brings a GROUP of 4 consecutive tile rows (4 x 256 B), row
// after row; groups are 1040 bytes apart (1024 + 16 of padding).  Hence, in elements,
//
//     offset(row, col) = (row >> 2) * 520 + (row & 3) * 128 + col
//
// How the LDS serves a 16-byte read (measured on gfx950): the two halves of the wavefront
// go separately; within a half of 32 lanes, lanes whose index has an even number of ones in
// bits 2, 3 and 4 (lanes 0-3, 12-15, 20-27) are served together, and so are the other 16.
// Each such set must touch every one of the 64 banks once (a lane covers 4 consecutive
// banks).  A pattern where lane i + 16 is a multiple of 256 bytes away from lane i, and lanes
// 0..15 cover 16 different 16-byte slots modulo 256 bytes, satisfies that.  Here lanes 0..15
// read the same chunk of rows 4*i + b (b fixed): 1040 bytes apart, i.e. one slot apart modulo
// 256; lanes 16..31 read row 4*i + b + 1, exactly 256 bytes further.  For that, row rho
// (0..31) of a 32-row MFMA operand of sub-tile kt (0/1) is tile row
// 4*(rho & 15) + (rho >> 4) + 2*kt.
#pragma once
#include "ody_common.h"

namespace tile128 {

constexpr int ROWS = 64;
constexpr int GROUP_ELEMS = 520;                 // 1040 bytes
constexpr int TILE_ELEMS = 16 * GROUP_ELEMS;     // 8320 elements = 16640 bytes
constexpr int TILE_BYTES = TILE_ELEMS * 2;

// tile row of MFMA row rho of sub-tile kt
__device__ __forceinline__ int tile_row(int rho, int kt) { return 4 * (rho & 15) + (rho >> 4) + 2 * kt; }

// tile row held in accumulator register r of lane group g (accumulator rows are
// rho = 8*(r>>2) + 4g + (r&3))
__device__ __forceinline__ int acc_tile_row(int r, int g, int kt) {
  return 32 * ((r >> 2) & 1) + 16 * g + 4 * (r & 3) + (r >> 3) + 2 * kt;
}

typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef __attribute__((address_space(1))) const void* global_void_ptr;

// Issues this thread's share of the direct loads of one 64 x 128 tile: 4 loads of
// 16 bytes (256 threads).  `base` points at row 0 of the matrix for this (batch, head);
// rows at or beyond `nrows` re-read row nrows-1 (finite filler that the caller masks).
__device__ __forceinline__ void load_tile_async(bf16* lds_tile, const bf16* base, int64_t row_stride, int row0,
                                                int nrows, int wave, int lane) {
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int grp = 4 * j + wave;
    int row = row0 + 4 * grp + (lane >> 4);
    row = row < nrows ? row : nrows - 1;
    const bf16* src = base + (int64_t)row * row_stride + 8 * (lane & 15);
    __builtin_amdgcn_global_load_lds((global_void_ptr)src, (lds_void_ptr)(lds_tile + grp * GROUP_ELEMS), 16, 0, 0);
  }
}

// Per-lane element offset of the row-wise operand: MFMA row i, k = 8g..8g+7 of k-step 0,
// sub-tile 0.  Add ks*16 + kt*KT_ELEMS elements for k-step ks of sub-tile kt.
constexpr int KT_ELEMS = 256;                    // sub-tile 1 starts two rows further
__device__ __forceinline__ int row_frag_base(int g, int i) { return (i & 15) * GROUP_ELEMS + (i >> 4) * 128 + g * 8; }

__device__ __forceinline__ bf16x8 row_frag(const bf16* tile, int base, int ks, int kt) {
  return *reinterpret_cast<const bf16x8*>(tile + base + ks * 16 + kt * KT_ELEMS);
}

// ---------------------------------------------------------------------------------
// Transposed tiles ("images").  An operand that an MFMA contracts over its ROW index
// (V in O^T += V^T P^T, Q and dO in the dK/dV products, K in dQ^T += K^T dS^T) is not
// read with the transpose instruction -- ds_read_b64_tr_b16 delivers half the LDS
// bandwidth of a 16-byte read -- but from a transposed copy that a small pre-pass
// writes to the workspace, one 16 KB image per 64-row tile, already in the order the
// LDS wants:  128 image rows (the head-dim index d) x 8 chunks of 8 tile rows.
//
//   chunk c = 4*kt + 2*ss + g, element j   <->   tile row 32*(j>>2) + 16*g + 4*(j&3) + ss + 2*kt
//
// which is exactly the order in which lane group g holds the 8 contraction values of
// k-step ss of sub-tile kt in an accumulator (acc_tile_row).  Inside the image, chunks
// are stored chunk-major in groups of 16 image rows:
//
//   byte offset(d, c) = (d >> 4) * 2048 + c * 256 + (d & 15) * 16
//
// so the 16 lanes that are served together (16 consecutive d, same c) read 256
// contiguous bytes: all 64 banks, no padding.  The image is contiguous in global
// memory and in LDS, so the direct loads are plain 1 KB copies.
constexpr int IMG_ELEMS = 128 * 64;          // 16384 bytes
constexpr int IMG_BYTES = IMG_ELEMS * 2;

// position (chunk * 8 + element) of tile row `row` (0..63) inside an image row
__host__ __device__ __forceinline__ int image_pos(int row) {
  const int kt = (row >> 1) & 1, ss = row & 1, g = (row >> 4) & 1, j = 4 * (row >> 5) + ((row >> 2) & 3);
  return 8 * (4 * kt + 2 * ss + g) + j;
}

__device__ __forceinline__ void load_image_async(bf16* lds_img, const bf16* img, int wave, int lane) {
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int off = ((4 * j + wave) * 64 + lane) * 8;
    __builtin_amdgcn_global_load_lds((global_void_ptr)(img + off), (lds_void_ptr)(lds_img + (4 * j + wave) * 512), 16,
                                     0, 0);
  }
}

// Per-lane element offset of the A operand read from an image: MFMA row i <-> d = 32*dt + i.
// Add dt*2048 + (4*kt + 2*ss)*128 elements.
__device__ __forceinline__ int image_frag_base(int g, int i) { return (i >> 4) * 1024 + (i & 15) * 8 + g * 128; }

__device__ __forceinline__ bf16x8 image_frag(const bf16* img, int base, int dt, int ss, int kt) {
  return *reinterpret_cast<const bf16x8*>(img + base + dt * 2048 + (4 * kt + 2 * ss) * 128);
}

}  // namespace tile128

// The lane id, recomputed on the spot.  Where every register is spoken for, values derived from
// it are cheaper to rebuild than to keep (the alternative is a spill to scratch memory, whose
// reload then waits behind the tile loads in flight).
__device__ __forceinline__ int fresh_lane() {
  int ln;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
  return ln;
}

// Two wavefronts of a workgroup share each SIMD.  Started together and re-aligned by every
// workgroup barrier they run in lockstep -- both in their matrix phase, then both in their
// vector phase -- and the matrix pipe idles half of the time.  Raising the priority of the
// first wavefront to arrive on each SIMD breaks the symmetry: it runs ahead, and the other
// one fills the matrix pipe while the first is in its vector phase.
// Order of arrival of this wavefront among those of its workgroup on the same SIMD (0, 1, ...).
__device__ __forceinline__ int simd_rank(int tid) {
  __shared__ int simd_count[4];
  if (tid < 4) simd_count[tid] = 0;
  __syncthreads();
  const int simd = __builtin_amdgcn_s_getreg((1 << 11) | (4 << 6) | 4) & 3;   // HW_ID.SIMD_ID
  int rank = 0;
  if ((tid & 63) == 0) rank = atomicAdd(&simd_count[simd], 1);
  return __builtin_amdgcn_readfirstlane(rank);
}
__device__ __forceinline__ void simd_stagger(int tid) {
  if (simd_rank(tid) == 0) __builtin_amdgcn_s_setprio(2);
}

// Swap of the two wavefront halves through v_permlane32_swap: returns, in every lane,
// op(x of this lane, x of the lane 32 away).
__device__ __forceinline__ float half_swap_max(float x) {
  const unsigned u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float x) {
  const unsigned u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
