// Pre-pass of the head_dim-128 attention kernels: writes the transposed 64-row tile
// images (see attn_tile.h) of a (B, L, H, 128) bf16 matrix into the workspace.
// Memory-bound: every element is read once and written once, both with 16-byte accesses.
#include "attn_params.h"
#include "attn_tile.h"

namespace {

using namespace tile128;

// an image leaves by a streaming store: this kernel does not read it again
__device__ __forceinline__ void store_image_chunk(bf16* p, bf16x8 v) {
  typedef unsigned raw_t __attribute__((ext_vector_type(4)));
  __builtin_nontemporal_store(__builtin_bit_cast(raw_t, v), reinterpret_cast<raw_t*>(p));
}

// 16-byte chunk q of a tile's image, from the row-major copy of the tile in LDS (pitch 128 + 8): column
// d = 16 (q >> 7) + (q & 15), and with c = (q >> 4) & 7 the rows 32 (e >> 2) + 4 (e & 3) + r0, e = 0..7, where
// r0 = 16 (c & 1) + ((c >> 1) & 1) + 2 (c >> 2).  The 16 lanes of a transposing LDS read share c and the 16-column
// block: lane 4 k + m points at row r0 + 4 k, columns 4 m .. 4 m + 3 of the block, and receives rows r0 + 4 k',
// k' = 0..3, of column (its lane & 15) -- half a chunk per read instead of one element.
__device__ __forceinline__ bf16x8 image_chunk(const bf16* tile, int q) {
  constexpr int PITCH = 128 + 8;
  const int c = (q >> 4) & 7, l = q & 15;
  const int r0 = 16 * (c & 1) + ((c >> 1) & 1) + 2 * (c >> 2);
  const bf16* p = tile + (r0 + 4 * (l >> 2)) * PITCH + 16 * (q >> 7) + 4 * (l & 3);
  return concat4(lds_read_tr16(p), lds_read_tr16(p + 32 * PITCH));
}

__global__ __launch_bounds__(256) void attn_images_kernel(const bf16* __restrict__ src, AttnStrides s, int L,
                                                          bf16* __restrict__ dst, int ntiles, int H,
                                                          int* __restrict__ flags, int nflags) {
  constexpr int PITCH = 128 + 8;
  __shared__ __attribute__((aligned(16))) bf16 tile[64 * PITCH];
  const int tid = threadIdx.x;
  const int t = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  if (flags != nullptr && t == 0 && h == 0 && b == 0)
    for (int k = tid; k < nflags; k += 256) flags[k] = 0;
  const bf16* base = src + b * s.b + h * s.h;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int c = tid + 256 * j, row = c >> 4, col = (c & 15) * 8, gr = t * 64 + row;
    bf16x8 v = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if (gr < L) v = *reinterpret_cast<const bf16x8*>(base + (int64_t)gr * s.l + col);
    *reinterpret_cast<bf16x8*>(tile + row * PITCH + col) = v;
  }
  __syncthreads();
  bf16* img = dst + (((int64_t)b * H + h) * ntiles + t) * IMG_ELEMS;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    store_image_chunk(img + (tid + 256 * j) * 8, image_chunk(tile, tid + 256 * j));
  }
}

// The whole query side of the head_dim-128 backward in one pass over Q, dO and O (one block per 64-query tile of a
// head): delta = sum_d dO * O, the transposed images of the Q tile and of the dO tile, and the tile's start values
// (-lse / scale and -delta in the order of the dK/dV kernel's accumulator registers; layout described where that
// kernel reads them).  Replaces four launches that each went over the same rows.
__global__ __launch_bounds__(256) void attn_bwd_prepass_kernel(const AttnParams p, bf16* __restrict__ qimg,
                                                               bf16* __restrict__ doimg, bf16* __restrict__ stats) {
  constexpr int PITCH = 128 + 8;
  __shared__ __attribute__((aligned(16))) bf16 tq[64 * PITCH];
  __shared__ __attribute__((aligned(16))) bf16 tdo[64 * PITCH];
  __shared__ float sdelta[64];
  const int tid = threadIdx.x;
  const int t = blockIdx.x, h = blockIdx.y, b = blockIdx.z, ntiles = gridDim.x;
  const bf16* qb = static_cast<const bf16*>(p.q) + b * p.sq.b + h * p.sq.h;
  const bf16* dob = static_cast<const bf16*>(p.dout) + b * p.sdo.b + h * p.sdo.h;
  const bf16* ob = static_cast<const bf16*>(p.out) + b * p.so.b + h * p.so.h;
  const bf16x8 zero = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int c = tid + 256 * j, row = c >> 4, col = (c & 15) * 8, gr = t * 64 + row;
    bf16x8 qv = zero, dv = zero, ov = zero;
    if (gr < p.Lq) {
      qv = *reinterpret_cast<const bf16x8*>(qb + (int64_t)gr * p.sq.l + col);
      dv = *reinterpret_cast<const bf16x8*>(dob + (int64_t)gr * p.sdo.l + col);
      ov = *reinterpret_cast<const bf16x8*>(ob + (int64_t)gr * p.so.l + col);
    }
    *reinterpret_cast<bf16x8*>(tq + row * PITCH + col) = qv;
    *reinterpret_cast<bf16x8*>(tdo + row * PITCH + col) = dv;
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) acc = fmaf((float)ov[e], (float)dv[e], acc);
#pragma unroll
    for (int sft = 8; sft > 0; sft >>= 1) acc += __shfl_xor(acc, sft, 64);   // the 16 lanes of one row
    if ((tid & 15) == 0) {
      sdelta[row] = acc;
      if (gr < p.Lq) p.delta[((int64_t)b * p.Hq + h) * p.Lq + gr] = acc;
    }
  }
  __syncthreads();
  const int64_t tile_id = ((int64_t)b * p.Hq + h) * ntiles + t;
#pragma unroll
  for (int which = 0; which < 2; which++) {
    const bf16* tile = which ? tdo : tq;
    bf16* img = (which ? doimg : qimg) + tile_id * IMG_ELEMS;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      store_image_chunk(img + (tid + 256 * j) * 8, image_chunk(tile, tid + 256 * j));
    }
  }
  if (tid < 128) {
    // fp32 table [sub-tile mt][0: -lse/scale, 1: -delta][lane group g][accumulator register r]
    const int mt = tid >> 6, which = (tid >> 5) & 1, g = (tid >> 4) & 1, r = tid & 15;
    const int row = acc_tile_row(r, g, mt), qi = t * 64 + row;
    float x;
    if (which == 0) {
      const float l = (qi < p.Lq) ? p.lse[((int64_t)b * p.Hq + h) * p.Lq + qi] : INFINITY;
      x = (l == INFINITY || l == -INFINITY) ? -1e30f : -l / p.scale;
    } else {
      x = (qi < p.Lq) ? -sdelta[row] : 0.f;
    }
    reinterpret_cast<float*>(stats)[tile_id * 256 + tid] = x;   // records of 1 KB
  }
}

}  // namespace

int ody_launch_attn_bwd_prepass(const AttnParams& p, void* qimg, void* doimg, void* stats, hipStream_t st) {
  dim3 grid((p.Lq + 63) / 64, p.Hq, p.B);
  ODY_LAUNCH("attn_bwd_prepass", st, attn_bwd_prepass_kernel, grid, dim3(256), 0, p, static_cast<bf16*>(qimg),
             static_cast<bf16*>(doimg), static_cast<bf16*>(stats));
  return ody_check_launch("attn_bwd_prepass");
}

size_t ody_attn_images_bytes(int B, int L, int H) {
  return (size_t)B * H * ((L + 63) / 64) * tile128::IMG_BYTES;
}

int ody_launch_attn_images(const void* src, const AttnStrides& s, int B, int L, int H, void* dst, int* flags,
                           int nflags, hipStream_t st) {
  const int ntiles = (L + 63) / 64;
  dim3 grid(ntiles, H, B);
  ODY_LAUNCH("attn_images", st, attn_images_kernel, grid, dim3(256), 0, static_cast<const bf16*>(src), s, L,
             static_cast<bf16*>(dst), ntiles, H, flags, nflags);
  return ody_check_launch("attn_images");
}
