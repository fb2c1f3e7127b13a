// extern "C" entry points for attention.
#include <cmath>
#include <mutex>
#include "attn_params.h"

// Library-owned scratch of ody_attn_fwd_noalloc: one copy per GPU, held from the moment the code
// object is loaded on that GPU until the process ends.  In host code this name is only a handle
// for hipGetSymbolAddress; the device address is looked up once per device (scratch_of_device).
static __device__ __align__(256) unsigned char scratch[ODY_ATTN_FWD_NOALLOC_SCRATCH_BYTES];

namespace {

int check_common(const char* who, int B, int Lq, int Lk, int Hq, int Hkv, int D, int dtype) {
  ODY_REQUIRE(B > 0 && Lq > 0 && Lk > 0 && Hq > 0 && Hkv > 0, ODY_ERR_BAD_SHAPE,
              "%s: sizes must be positive (B=%d Lq=%d Lk=%d Hq=%d Hkv=%d)", who, B, Lq, Lk, Hq, Hkv);
  ODY_REQUIRE(Hq % Hkv == 0, ODY_ERR_BAD_SHAPE, "%s: Hq=%d is not a multiple of Hkv=%d", who, Hq, Hkv);
  ODY_REQUIRE(D == 64 || D == 128, ODY_ERR_UNSUPPORTED, "%s: head_dim %d not built (64, 128)", who, D);
  ODY_REQUIRE(dtype == ODY_BF16 || dtype == ODY_F32, ODY_ERR_UNSUPPORTED, "%s: dtype %d unknown", who, dtype);
  ODY_REQUIRE((int64_t)B * Hq * ((Lq + 63) / 64 + (Lk + 63) / 64) < (int64_t)1 << 31, ODY_ERR_BAD_SHAPE,
              "%s: too many blocks for one launch", who);
  return ODY_OK;
}

// All kernels move 16-byte vectors: pointers 16-byte aligned, strides multiples of 8 (bf16) or 4 (fp32) elements.
int check_tensor(const char* who, const char* name, const void* ptr, const AttnStrides& s, int dtype, bool vec) {
  ODY_REQUIRE(ptr != nullptr, ODY_ERR_NULL, "%s: %s is NULL", who, name);
  if (vec) {
    const int q = (dtype == ODY_BF16) ? 8 : 4;
    ODY_REQUIRE(ody_aligned16(ptr) && s.b % q == 0 && s.l % q == 0 && s.h % q == 0, ODY_ERR_MISALIGNED,
                "%s: %s needs a 16-byte aligned pointer and strides that are multiples of %d elements", who, name, q);
  }
  return ODY_OK;
}

}  // namespace

extern "C" size_t ody_attn_fwd_workspace_bytes(int B, int Lq, int Lk, int Hq, int Hkv, int D, int dtype);

namespace {
// p_drop in (0, 1): the dropout fields of the argument block; 0: none
int set_dropout(const char* who, AttnParams& p, float p_drop, uint64_t seed) {
  ODY_REQUIRE(p_drop >= 0.f && p_drop < 1.f, ODY_ERR_BAD_SHAPE, "%s: the dropout probability must be in [0, 1), got %g", who,
              (double)p_drop);
  if (p_drop == 0.f) return ODY_OK;
  const double t = (double)p_drop * 4294967296.0;
  p.drop_thresh = t >= 4294967295.0 ? 4294967295u : (t < 1.0 ? 1u : (unsigned)t);
  p.drop_seed = (unsigned)(seed ^ (seed >> 32));
  p.drop_scale = 1.f / (1.f - p_drop);
  return ODY_OK;
}

int attn_fwd_impl(const char* who, const void* q, const void* k, const void* v, void* out, float* lse,
                  int B, int Lq, int Lk, int Hq, int Hkv, int D,
                  int64_t sq_b, int64_t sq_l, int64_t sq_h,
                  int64_t sk_b, int64_t sk_l, int64_t sk_h,
                  int64_t sv_b, int64_t sv_l, int64_t sv_h,
                  int64_t so_b, int64_t so_l, int64_t so_h,
                  float scale, int causal, int dtype, void* workspace, size_t workspace_bytes,
                  void* stream, float p_drop, uint64_t seed) {
  int rc = check_common(who, B, Lq, Lk, Hq, Hkv, D, dtype);
  if (rc) return rc;
  AttnParams p{};
  if ((rc = set_dropout(who, p, p_drop, seed))) return rc;
  p.q = q; p.k = k; p.v = v; p.out = out; p.lse = lse;
  p.B = B; p.Lq = Lq; p.Lk = Lk; p.Hq = Hq; p.Hkv = Hkv; p.group = Hq / Hkv;
  p.causal = causal ? 1 : 0; p.off = Lk - Lq;
  p.scale = scale; p.scale_log2e = scale * ODY_LOG2E;
  p.sq = {sq_b, sq_l, sq_h}; p.sk = {sk_b, sk_l, sk_h}; p.sv = {sv_b, sv_l, sv_h}; p.so = {so_b, so_l, so_h};
  const bool vec = true;
  if ((rc = check_tensor(who, "q", q, p.sq, dtype, vec))) return rc;
  if ((rc = check_tensor(who, "k", k, p.sk, dtype, vec))) return rc;
  if ((rc = check_tensor(who, "v", v, p.sv, dtype, vec))) return rc;
  if ((rc = check_tensor(who, "out", out, p.so, dtype, vec))) return rc;
  ODY_REQUIRE(lse != nullptr, ODY_ERR_NULL, "%s: lse is NULL", who);
  ODY_REQUIRE(scale > 0.f && std::isfinite(scale), ODY_ERR_BAD_SHAPE, "%s: scale must be positive", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == ODY_BF16 && D == 128 && p.drop_thresh == 0) {
    // the least that will do: without room for the parts of a key-split call the call runs unsplit
    const size_t need = (ody_attn_fwd_w8_workspace(B, Lq, Lk, Hq, Hkv, false) + 255) & ~(size_t)255;
    ODY_REQUIRE(workspace != nullptr, ODY_ERR_NULL, "%s: workspace is NULL", who);
    ODY_REQUIRE(workspace_bytes >= need, ODY_ERR_WORKSPACE, "%s: workspace of %zu bytes, %zu needed", who,
                workspace_bytes, need);
    ODY_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, ODY_ERR_MISALIGNED,
                "%s: workspace must be 256-byte aligned", who);
    return ody_launch_attn_fwd_w8(p, workspace, workspace_bytes, st);
  }
  if (dtype == ODY_BF16) return ody_launch_attn_fwd_mfma(p, D, st);
  return ody_launch_attn_fwd_f32(p, D, st);
}
}  // namespace

extern "C" int ody_attn_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                            int B, int Lq, int Lk, int Hq, int Hkv, int D,
                            int64_t sq_b, int64_t sq_l, int64_t sq_h,
                            int64_t sk_b, int64_t sk_l, int64_t sk_h,
                            int64_t sv_b, int64_t sv_l, int64_t sv_h,
                            int64_t so_b, int64_t so_l, int64_t so_h,
                            float scale, int causal, int dtype, void* workspace, size_t workspace_bytes,
                            void* stream) {
  return attn_fwd_impl("ody_attn_fwd", q, k, v, out, lse, B, Lq, Lk, Hq, Hkv, D, sq_b, sq_l, sq_h, sk_b, sk_l, sk_h, sv_b, sv_l, sv_h,
                       so_b, so_l, so_h, scale, causal, dtype, workspace, workspace_bytes, stream, 0.f, 0);
}

extern "C" int ody_attn_fwd_dropout(const void* q, const void* k, const void* v, void* out, float* lse,
                                    int B, int Lq, int Lk, int Hq, int Hkv, int D,
                                    int64_t sq_b, int64_t sq_l, int64_t sq_h,
                                    int64_t sk_b, int64_t sk_l, int64_t sk_h,
                                    int64_t sv_b, int64_t sv_l, int64_t sv_h,
                                    int64_t so_b, int64_t so_l, int64_t so_h,
                                    float scale, int causal, int dtype, void* workspace, size_t workspace_bytes,
                                    void* stream, float p_drop, uint64_t seed) {
  return attn_fwd_impl("ody_attn_fwd_dropout", q, k, v, out, lse, B, Lq, Lk, Hq, Hkv, D, sq_b, sq_l, sq_h, sk_b, sk_l, sk_h, sv_b, sv_l,
                       sv_h, so_b, so_l, so_h, scale, causal, dtype, workspace, workspace_bytes, stream, p_drop, seed);
}

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (each GPU holds its own copy at its own address).
int scratch_of_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  ODY_REQUIRE(e == hipSuccess && dev >= 0 && dev < kMaxDevices, ODY_ERR_LAUNCH,
              "ody_attn_fwd_noalloc: no usable current device (%s)", hipGetErrorString(e));
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    ODY_REQUIRE(e == hipSuccess && ptr != nullptr, ODY_ERR_LAUNCH,
                "ody_attn_fwd_noalloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return ODY_OK;
}
}  // namespace

extern "C" int ody_attn_fwd_noalloc(const void* q, const void* k, const void* v, void* out, float* lse,
                                    int B, int Lq, int Lk, int Hq, int Hkv, int D,
                                    int64_t sq_b, int64_t sq_l, int64_t sq_h,
                                    int64_t sk_b, int64_t sk_l, int64_t sk_h,
                                    int64_t sv_b, int64_t sv_l, int64_t sv_h,
                                    int64_t so_b, int64_t so_l, int64_t so_h,
                                    float scale, int causal, int dtype, void* stream) {
  int rc = check_common("ody_attn_fwd_noalloc", B, Lq, Lk, Hq, Hkv, D, dtype);
  if (rc) return rc;
  // the fixed scratch holds the flags and the V images, and the parts of a call that cuts its key ranges if they fit
  // as well (then the result is that of ody_attn_fwd bit for bit); otherwise such a call runs unsplit here
  size_t need = 0;
  if (dtype == ODY_BF16 && D == 128) {
    need = (ody_attn_fwd_w8_workspace(B, Lq, Lk, Hq, Hkv, true) + 255) & ~(size_t)255;
    if (need > (size_t)ODY_ATTN_FWD_NOALLOC_SCRATCH_BYTES)
      need = (ody_attn_fwd_w8_workspace(B, Lq, Lk, Hq, Hkv, false) + 255) & ~(size_t)255;
  }
  ODY_REQUIRE(need <= (size_t)ODY_ATTN_FWD_NOALLOC_SCRATCH_BYTES, ODY_ERR_WORKSPACE,
              "ody_attn_fwd_noalloc: this shape needs %zu bytes of scratch, the library-owned buffer holds %zu "
              "(256 bytes per key row of every kv head: B*Hkv*Lk <= about 131000); use ody_attn_fwd with a "
              "caller workspace", need, (size_t)ODY_ATTN_FWD_NOALLOC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (need > 0 && (rc = scratch_of_device(&ws))) return rc;
  return ody_attn_fwd(q, k, v, out, lse, B, Lq, Lk, Hq, Hkv, D, sq_b, sq_l, sq_h, sk_b, sk_l, sk_h, sv_b, sv_l, sv_h,
                      so_b, so_l, so_h, scale, causal, dtype, ws, need, stream);
}

extern "C" size_t ody_attn_fwd_workspace_bytes(int B, int Lq, int Lk, int Hq, int Hkv, int D, int dtype) {
  if (B <= 0 || Lq <= 0 || Lk <= 0 || Hq <= 0 || Hkv <= 0) return 0;
  if (dtype == ODY_BF16 && D == 128) return (ody_attn_fwd_w8_workspace(B, Lq, Lk, Hq, Hkv, true) + 255) & ~(size_t)255;
  return 0;
}

namespace {
size_t delta_bytes(int B, int Lq, int Hq) { return ((size_t)B * Lq * Hq * sizeof(float) + 255) & ~(size_t)255; }
}

extern "C" size_t ody_attn_bwd_workspace_bytes(int B, int Lq, int Lk, int Hq, int Hkv, int D, int dtype) {
  if (B <= 0 || Lq <= 0 || Lk <= 0 || Hq <= 0 || Hkv <= 0) return 0;
  size_t n = delta_bytes(B, Lq, Hq);
  if (dtype == ODY_BF16 && D == 128) n += ody_attn_bwd_pipe_workspace(B, Lq, Lk, Hq, Hkv);
  return n;
}

extern "C" size_t ody_attn_bwd_ds_bytes(int B, int Lq, int Lk, int Hq, int Hkv, int D, int dtype, int causal) {
  if (B <= 0 || Lq <= 0 || Lk <= 0 || Hq <= 0 || Hkv <= 0 || dtype != ODY_BF16 || D != 128) return 0;
  return (ody_attn_bwd_pipe_ds_bytes(B, Lq, Lk, Hq, causal) + 255) & ~(size_t)255;
}

namespace {
int attn_bwd_impl(const char* who, const void* rope_q, const void* rope_k,
                  const void* q, const void* k, const void* v, const void* out, const float* lse,
                  const void* dout, void* dq, void* dk, void* dv,
                  int B, int Lq, int Lk, int Hq, int Hkv, int D,
                  int64_t sq_b, int64_t sq_l, int64_t sq_h,
                  int64_t sk_b, int64_t sk_l, int64_t sk_h,
                  int64_t sv_b, int64_t sv_l, int64_t sv_h,
                  int64_t so_b, int64_t so_l, int64_t so_h,
                  int64_t sdo_b, int64_t sdo_l, int64_t sdo_h,
                  int64_t sdq_b, int64_t sdq_l, int64_t sdq_h,
                  int64_t sdk_b, int64_t sdk_l, int64_t sdk_h,
                  int64_t sdv_b, int64_t sdv_l, int64_t sdv_h,
                  float scale, int causal, int flags, int dtype,
                  void* workspace, size_t workspace_bytes, void* stream, float p_drop = 0.f, uint64_t seed = 0) {
  int rc = check_common(who, B, Lq, Lk, Hq, Hkv, D, dtype);
  if (rc) return rc;
  ODY_REQUIRE((flags & ~(ODY_BWD_ACCUMULATE_DQ | ODY_BWD_DQ_F32 | ODY_BWD_REUSE_QUERY_SIDE | ODY_BWD_KEEP_DS)) == 0, ODY_ERR_UNSUPPORTED,
              "%s: unknown flag bits in %d", who, flags);
  AttnParams p{};
  if ((rc = set_dropout(who, p, p_drop, seed))) return rc;
  ODY_REQUIRE(p.drop_thresh == 0 || !(flags & ODY_BWD_KEEP_DS), ODY_ERR_UNSUPPORTED,
              "%s: ODY_BWD_KEEP_DS is not available with dropout", who);
  ODY_REQUIRE(p.drop_thresh == 0 || !(rope_q || rope_k), ODY_ERR_UNSUPPORTED, "%s: no rotary tables with dropout", who);
  p.q = q; p.k = k; p.v = v; p.out = const_cast<void*>(out); p.lse = const_cast<float*>(lse);
  p.dout = dout; p.dq = dq; p.dk = dk; p.dv = dv;
  p.B = B; p.Lq = Lq; p.Lk = Lk; p.Hq = Hq; p.Hkv = Hkv; p.group = Hq / Hkv;
  p.causal = causal ? 1 : 0; p.off = Lk - Lq; p.accumulate_dq = (flags & ODY_BWD_ACCUMULATE_DQ) ? 1 : 0;
  p.dq_f32 = (flags & ODY_BWD_DQ_F32) || dtype == ODY_F32 ? 1 : 0;
  p.reuse_query_side = (flags & ODY_BWD_REUSE_QUERY_SIDE) ? 1 : 0;
  p.scale = scale; p.scale_log2e = scale * ODY_LOG2E;
  p.sq = {sq_b, sq_l, sq_h}; p.sk = {sk_b, sk_l, sk_h}; p.sv = {sv_b, sv_l, sv_h}; p.so = {so_b, so_l, so_h};
  p.sdo = {sdo_b, sdo_l, sdo_h}; p.sdq = {sdq_b, sdq_l, sdq_h}; p.sdk = {sdk_b, sdk_l, sdk_h};
  p.sdv = {sdv_b, sdv_l, sdv_h};
  const bool vec = true;
  if ((rc = check_tensor(who, "q", q, p.sq, dtype, vec))) return rc;
  if ((rc = check_tensor(who, "k", k, p.sk, dtype, vec))) return rc;
  if ((rc = check_tensor(who, "v", v, p.sv, dtype, vec))) return rc;
  if ((rc = check_tensor(who, "out", out, p.so, dtype, vec))) return rc;
  if ((rc = check_tensor(who, "dout", dout, p.sdo, dtype, vec))) return rc;
  if ((rc = check_tensor(who, "dq", dq, p.sdq, p.dq_f32 ? ODY_F32 : dtype, vec))) return rc;
  if ((rc = check_tensor(who, "dk", dk, p.sdk, dtype, vec))) return rc;
  if ((rc = check_tensor(who, "dv", dv, p.sdv, dtype, vec))) return rc;
  ODY_REQUIRE(lse != nullptr, ODY_ERR_NULL, "%s: lse is NULL", who);
  ODY_REQUIRE(scale > 0.f && std::isfinite(scale), ODY_ERR_BAD_SHAPE, "%s: scale must be positive", who);
  ODY_REQUIRE(workspace != nullptr, ODY_ERR_NULL, "%s: workspace is NULL", who);
  const size_t ws_base = ody_attn_bwd_workspace_bytes(B, Lq, Lk, Hq, Hkv, D, dtype);
  size_t ws_ds = 0;
  if (flags & ODY_BWD_KEEP_DS) {
    ws_ds = ody_attn_bwd_ds_bytes(B, Lq, Lk, Hq, Hkv, D, dtype, causal);
    ODY_REQUIRE(ws_ds > 0, ODY_ERR_UNSUPPORTED,
                "%s: ODY_BWD_KEEP_DS needs bf16, head_dim 128, Lq and Lk multiples of 256 and, if causal, Lq == Lk", who);
  }
  ODY_REQUIRE(workspace_bytes >= ws_base + ws_ds, ODY_ERR_WORKSPACE, "%s: workspace of %zu bytes, %zu needed", who,
              workspace_bytes, ws_base + ws_ds);
  ODY_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, ODY_ERR_MISALIGNED,
              "%s: workspace must be 256-byte aligned", who);
  if (rope_q || rope_k) {
    ODY_REQUIRE(rope_q && rope_k, ODY_ERR_NULL, "%s: both tables or none", who);
    ODY_REQUIRE(dtype == ODY_BF16 && D == 128, ODY_ERR_UNSUPPORTED, "%s: the rotary tables need bf16 and head_dim 128", who);
    ODY_REQUIRE(!p.dq_f32 && !p.accumulate_dq, ODY_ERR_UNSUPPORTED,
                "%s: the rotary tables cannot be combined with an accumulated or fp32 dq", who);
    ODY_REQUIRE(ody_aligned16(rope_q) && ody_aligned16(rope_k), ODY_ERR_MISALIGNED, "%s: tables must be 16-byte aligned", who);
    p.rope_q = static_cast<const bf16*>(rope_q);
    p.rope_k = static_cast<const bf16*>(rope_k);
  }
  p.delta = static_cast<float*>(workspace);
  if (ws_ds) p.ds = reinterpret_cast<bf16*>(static_cast<char*>(workspace) + ws_base);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == ODY_BF16 && D == 128 && p.drop_thresh == 0)   // its query-side pre-pass computes delta as well
    return ody_launch_attn_bwd_pipe(p, static_cast<char*>(workspace) + delta_bytes(B, Lq, Hq), st);
  if (!p.reuse_query_side && (rc = ody_launch_attn_delta(p, D, dtype, st))) return rc;
  if (dtype == ODY_BF16) return ody_launch_attn_bwd_mfma(p, D, st);
  return ody_launch_attn_bwd_f32(p, D, st);
}
}  // namespace

extern "C" int ody_attn_bwd(const void* q, const void* k, const void* v, const void* out, const float* lse,
                            const void* dout, void* dq, void* dk, void* dv,
                            int B, int Lq, int Lk, int Hq, int Hkv, int D,
                            int64_t sq_b, int64_t sq_l, int64_t sq_h,
                            int64_t sk_b, int64_t sk_l, int64_t sk_h,
                            int64_t sv_b, int64_t sv_l, int64_t sv_h,
                            int64_t so_b, int64_t so_l, int64_t so_h,
                            int64_t sdo_b, int64_t sdo_l, int64_t sdo_h,
                            int64_t sdq_b, int64_t sdq_l, int64_t sdq_h,
                            int64_t sdk_b, int64_t sdk_l, int64_t sdk_h,
                            int64_t sdv_b, int64_t sdv_l, int64_t sdv_h,
                            float scale, int causal, int flags, int dtype,
                            void* workspace, size_t workspace_bytes, void* stream) {
  return attn_bwd_impl("ody_attn_bwd", nullptr, nullptr, q, k, v, out, lse, dout, dq, dk, dv, B, Lq, Lk, Hq, Hkv, D, sq_b, sq_l, sq_h, sk_b, sk_l, sk_h, sv_b, sv_l, sv_h,
                       so_b, so_l, so_h, sdo_b, sdo_l, sdo_h, sdq_b, sdq_l, sdq_h, sdk_b, sdk_l, sdk_h, sdv_b, sdv_l, sdv_h, scale,
                       causal, flags, dtype, workspace, workspace_bytes, stream);
}

extern "C" int ody_attn_bwd_dropout(const void* q, const void* k, const void* v, const void* out, const float* lse,
                                    const void* dout, void* dq, void* dk, void* dv,
                                    int B, int Lq, int Lk, int Hq, int Hkv, int D,
                                    int64_t sq_b, int64_t sq_l, int64_t sq_h,
                                    int64_t sk_b, int64_t sk_l, int64_t sk_h,
                                    int64_t sv_b, int64_t sv_l, int64_t sv_h,
                                    int64_t so_b, int64_t so_l, int64_t so_h,
                                    int64_t sdo_b, int64_t sdo_l, int64_t sdo_h,
                                    int64_t sdq_b, int64_t sdq_l, int64_t sdq_h,
                                    int64_t sdk_b, int64_t sdk_l, int64_t sdk_h,
                                    int64_t sdv_b, int64_t sdv_l, int64_t sdv_h,
                                    float scale, int causal, int flags, int dtype,
                                    void* workspace, size_t workspace_bytes, void* stream, float p_drop, uint64_t seed) {
  return attn_bwd_impl("ody_attn_bwd_dropout", nullptr, nullptr, q, k, v, out, lse, dout, dq, dk, dv, B, Lq, Lk, Hq, Hkv, D, sq_b, sq_l,
                       sq_h, sk_b, sk_l, sk_h, sv_b, sv_l, sv_h, so_b, so_l, so_h, sdo_b, sdo_l, sdo_h, sdq_b, sdq_l, sdq_h, sdk_b,
                       sdk_l, sdk_h, sdv_b, sdv_l, sdv_h, scale, causal, flags, dtype, workspace, workspace_bytes, stream, p_drop,
                       seed);
}

extern "C" int ody_attn_bwd_rope(const void* q, const void* k, const void* v, const void* out, const float* lse,
                            const void* dout, void* dq, void* dk, void* dv,
                            int B, int Lq, int Lk, int Hq, int Hkv, int D,
                            int64_t sq_b, int64_t sq_l, int64_t sq_h,
                            int64_t sk_b, int64_t sk_l, int64_t sk_h,
                            int64_t sv_b, int64_t sv_l, int64_t sv_h,
                            int64_t so_b, int64_t so_l, int64_t so_h,
                            int64_t sdo_b, int64_t sdo_l, int64_t sdo_h,
                            int64_t sdq_b, int64_t sdq_l, int64_t sdq_h,
                            int64_t sdk_b, int64_t sdk_l, int64_t sdk_h,
                            int64_t sdv_b, int64_t sdv_l, int64_t sdv_h,
                            float scale, int causal, int flags, int dtype,
                            void* workspace, size_t workspace_bytes, void* stream,
                            const void* rope_table_q, const void* rope_table_k) {
  ODY_REQUIRE(rope_table_q && rope_table_k, ODY_ERR_NULL, "ody_attn_bwd_rope: rotary table is NULL");
  return attn_bwd_impl("ody_attn_bwd_rope", rope_table_q, rope_table_k, q, k, v, out, lse, dout, dq, dk, dv, B, Lq, Lk, Hq, Hkv, D, sq_b, sq_l, sq_h, sk_b, sk_l, sk_h, sv_b, sv_l, sv_h,
                       so_b, so_l, so_h, sdo_b, sdo_l, sdo_h, sdq_b, sdq_l, sdq_h, sdk_b, sdk_l, sdk_h, sdv_b, sdv_l, sdv_h, scale,
                       causal, flags, dtype, workspace, workspace_bytes, stream);
}
