// Pre-pass of the head_dim-128 attention kernels: writes the transposed 64-row tile
// images (see attn_tile.h) of a (B, L, H, 128) bf16 matrix into the workspace.
// Memory-bound: every element is read once and written once, both with 16-byte accesses.
#include "attn_params.h"
#include "attn_tile.h"

namespace {

using namespace tile128;

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
    const int q = tid + 256 * j;                    // 16-byte chunk of the image
    const int d = 16 * (q >> 7) + (q & 15), c = (q >> 4) & 7;
    const int kt = c >> 2, ss = (c >> 1) & 1, g = c & 1;
    bf16x8 v;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int row = 32 * (e >> 2) + 16 * g + 4 * (e & 3) + ss + 2 * kt;
      v[e] = tile[row * PITCH + d];
    }
    *reinterpret_cast<bf16x8*>(img + q * 8) = v;
  }
}

}  // namespace

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
