// Argument block shared by the attention kernels (forward, backward, SIMT fp32).
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
  float scale;        // softmax scale
  float scale_log2e;  // scale * log2(e)
  AttnStrides sq, sk, sv, so, sdo, sdq, sdk, sdv;
};

// Launchers (one per translation unit); each returns an ody_status.
int ody_launch_attn_fwd_mfma(const AttnParams& p, int D, hipStream_t st);
int ody_launch_attn_bwd_mfma(const AttnParams& p, int D, hipStream_t st);
int ody_launch_attn_fwd_simt(const AttnParams& p, int D, int dtype, hipStream_t st);
int ody_launch_attn_bwd_simt(const AttnParams& p, int D, int dtype, hipStream_t st);
int ody_launch_attn_delta(const AttnParams& p, int D, int dtype, hipStream_t st);
