// Argument block shared by the attention kernels (forward, backward, bf16 and fp32).
#pragma once
#include "ody_common.h"

struct AttnStrides {
  int64_t b, l, h;  // elements; head_dim stride is 1
};

struct AttnParams {
  const void* q;
  const void* k;
  const void* v;
  void* out;          // fwd: written; bwd: read
  float* lse;         // fwd: written; bwd: read            (B, Hq, Lq)
  const void* dout;   // bwd
  void* dq;           // bwd
  void* dk;           // bwd
  void* dv;           // bwd
  float* delta;       // bwd workspace: sum_d dO*O          (B, Hq, Lq)
  int B, Lq, Lk, Hq, Hkv, group;
  int causal;         // 0/1
  int off;            // Lk - Lq: key j visible to query i iff j <= i + off
  int accumulate_dq;  // bwd: dq += result
  int dq_f32;         // bwd: dq is an fp32 buffer (strides in fp32 elements) whatever the storage type of q
  int reuse_query_side;  // bwd: delta, start values and the Q / dO images in the workspace are those of the previous call
  // bwd, bf16 head_dim 128 only: cos / sin tables (ody_rope_table layout, row pitch 128) of the query rows (B * Lq) and
  // of the key rows (B * Lk); when set, dq and dk leave the kernels rotated back by the negative angle, i.e. as the
  // gradient of the projection BEFORE its rotary embedding
  const bf16* rope_q;
  const bf16* rope_k;
  // bwd, bf16 head_dim 128, Lq and Lk multiples of 256 (causal: Lq == Lk): when set, the dK/dV kernel keeps
  // every dS tile here (ody_attn_bwd_ds_bytes) and dQ is computed from them instead of from a second pass over S and dP
  bf16* ds;
  // attention dropout (bf16, the kernels of attn_fwd_mfma.hip / attn_bwd_mfma.hip only): an entry of P is dropped when
  // its 32-bit hash (ody_dropout_hash) is below drop_thresh = p * 2^32; kept entries are scaled by drop_scale =
  // 1 / (1 - p).  drop_thresh == 0: no dropout.
  unsigned drop_thresh, drop_seed;
  float drop_scale;
  float scale;        // softmax scale
  float scale_log2e;  // scale * log2(e)
  AttnStrides sq, sk, sv, so, sdo, sdq, sdk, sdv;
};

// Block order of the attention kernels: a 1-D grid whose linear id runs over (head, batch)
// fastest and over the row-block rank slowest.  With causal masking the work of a row block
// grows with its index, so rank 0 is the heaviest block: the dispatcher then hands out the
// heavy blocks of ALL heads first and the light ones fill the tail (a (blocks, heads) grid
// would start with every block of head 0, light ones included).  Consecutive ids also map
// to consecutive XCDs, so with 4 or 8 heads each XCD works on one head and its workgroups
// walk the same K / V (or Q / dO) tiles at the same time, sharing them through its L2.
struct BlockCoord { int rank, h, b; };
#ifdef __HIPCC__
__device__ __forceinline__ BlockCoord ody_block_coord_of(int id, int H, int B) {
  const int hb = id % (H * B);
  return BlockCoord{id / (H * B), hb % H, hb / H};
}
__device__ __forceinline__ BlockCoord ody_block_coord(int H, int B) { return ody_block_coord_of(blockIdx.x, H, B); }

// The dropout decision of score (batch b, query head h, query q, key k): a counter-based hash, so that the forward
// kernel and both backward kernels, which hold the scores in different layouts, agree without exchanging anything.
//   head value  u = mix(seed ^ (b * Hq + h) * 0x85ebca77)        (once per block)
//   row value   r = mix(u + q * 0x9e3779b1)                      (once per query)
//   hash        x = mix(r ^ k * 0xc2b2ae3d);  the score is kept iff x >= thresh
// mix is the 32-bit finalizer of MurmurHash3.  tests/ restate it in integer arithmetic on the host.
__device__ __forceinline__ unsigned ody_mix32(unsigned x) {
  x ^= x >> 16; x *= 0x85ebca6bu; x ^= x >> 13; x *= 0xc2b2ae35u; x ^= x >> 16;
  return x;
}
__device__ __forceinline__ unsigned ody_dropout_head(unsigned seed, int bh) { return ody_mix32(seed ^ ((unsigned)bh * 0x85ebca77u)); }
__device__ __forceinline__ unsigned ody_dropout_row(unsigned head, int q) { return ody_mix32(head + (unsigned)q * 0x9e3779b1u); }
__device__ __forceinline__ unsigned ody_dropout_hash(unsigned row, int k) { return ody_mix32(row ^ ((unsigned)k * 0xc2b2ae3du)); }
#endif

// Launchers (one per translation unit); each returns an ody_status.
int ody_launch_attn_fwd_mfma(const AttnParams& p, int D, hipStream_t st);
// transposed 64-row tile images of a (B, L, H, 128) bf16 matrix (attn_tile.h)
size_t ody_attn_images_bytes(int B, int L, int H);
// also zeroes `nflags` ints at `flags` (may be NULL)
int ody_launch_attn_images(const void* src, const AttnStrides& s, int B, int L, int H, void* dst, int* flags,
                           int nflags, hipStream_t st);
// head_dim 128 backward, everything that depends on the queries only, in one launch: p.delta, the transposed images
// of Q and dO and the start values (1 KB per 64-query tile)
int ody_launch_attn_bwd_prepass(const AttnParams& p, void* qimg, void* doimg, void* stats, hipStream_t st);
// head_dim 128 only, 8 wavefronts x 32 queries per block; workspace of ody_attn_fwd_w8_workspace(...) bytes.
// with_split: with room for the fp32 parts of a call whose fully visible key range is cut into 2 or 4 parts (few query
// blocks against many keys); a workspace without that room makes such a call run unsplit.
int ody_launch_attn_fwd_w8(const AttnParams& p, void* workspace, size_t workspace_bytes, hipStream_t st);
size_t ody_attn_fwd_w8_workspace(int B, int Lq, int Lk, int Hq, int Hkv, bool with_split);
// the online-rescaling forward kernel restricted to query blocks of `block` rows whose flag is set
int ody_launch_attn_fwd_mfma_flagged(const AttnParams& p, const int* flags, int block, hipStream_t st);
// head_dim 128 only; workspace of ody_attn_bwd_pipe_workspace(...) bytes (p.delta is set separately)
size_t ody_attn_bwd_pipe_workspace(int B, int Lq, int Lk, int Hq, int Hkv);
// bytes of the kept dS tiles (AttnParams::ds), 0 where the shape does not qualify
size_t ody_attn_bwd_pipe_ds_bytes(int B, int Lq, int Lk, int Hq, int causal);
int ody_launch_attn_bwd_pipe(const AttnParams& p, void* workspace, hipStream_t st);
int ody_launch_attn_bwd_mfma(const AttnParams& p, int D, hipStream_t st);
// fp32 on the fp32 matrix cores
int ody_launch_attn_fwd_f32(const AttnParams& p, int D, hipStream_t st);
int ody_launch_attn_bwd_f32(const AttnParams& p, int D, hipStream_t st);
int ody_launch_attn_delta(const AttnParams& p, int D, int dtype, hipStream_t st);
