/*
 * odysseus_hip.h -- C ABI of libodysseus_hip.so: the per-rank compute of the
 * Odysseus decoder layer as hand-written HIP kernels for gfx950 (MI355X).
 *
 * The reference has no FFI layer: its boundary is Python (nn.Module classes and
 * torch.autograd.Function.apply) over third-party kernels.  Each entry point
 * below replaces the third-party routine that a reference call site invokes;
 * the call site is cited next to it.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; the library never
 *     allocates, frees or keeps a pointer after the call returns;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*); no entry
 *     point synchronises the device;
 *   - `dtype` is ODY_BF16 (bf16 storage, fp32 accumulation, bf16 MFMA) or ODY_F32
 *     (fp32 storage and arithmetic, fp32 MFMA);
 *   - strides are in ELEMENTS; the innermost (head_dim / feature) stride is 1;
 *   - return value: 0 on success, a negative ody_status otherwise;
 *     ody_last_error() returns a thread-local message for the last failure.
 *     Nothing throws or aborts across this boundary.
 */
#ifndef ODYSSEUS_HIP_H
#define ODYSSEUS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum ody_dtype { ODY_BF16 = 0, ODY_F32 = 1 };

enum ody_status {
  ODY_OK = 0,
  ODY_ERR_BAD_SHAPE = -1,      /* non-positive size, Hq % Hkv != 0, ... */
  ODY_ERR_UNSUPPORTED = -2,    /* head_dim / dtype / flag combination not built */
  ODY_ERR_MISALIGNED = -3,     /* pointer or stride breaks the 16-byte rule */
  ODY_ERR_NULL = -4,           /* required pointer is NULL */
  ODY_ERR_WORKSPACE = -5,      /* workspace smaller than ody_*_workspace_bytes */
  ODY_ERR_LAUNCH = -6          /* hipLaunchKernel reported an error */
};

const char* ody_last_error(void);
int ody_version(void);

/* The current device as the kernels see it (no counterpart in the reference): compute units, the
 * engine clock in kHz and the LDS bytes of one compute unit.  Any pointer may be NULL.  The bf16
 * matrix peak follows as compute_units * clock * 4096 FLOP per clock (4 SIMDs, one 32x32x16 MFMA
 * per 32 cycles each).
 */
int ody_device_info(int* compute_units, int* clock_khz, int* lds_bytes_per_cu);

/* Per-kernel timer (no counterpart in the reference, whose only clock is time.time()
 * around whole steps, train.py:185-229).  While enabled, every kernel launch of the
 * library is bracketed by a pair of HIP events on its launch stream.
 * ody_profile_collect waits for the recorded events, writes one text line per kernel
 * name -- "name launches total_ms min_ms" -- into out (NUL-terminated, at most cap
 * bytes) and forgets them.
 */
int ody_profile_enable(int on);
int ody_profile_collect(char* out, size_t cap);

/* ---- attention ---------------------------------------------------------
 * Replaces flash_attn_func(q, k, v, dropout_p=0, softmax_scale, causal) as
 * reached from decoder/odysseus.py:256-263 (via HF _flash_attention_forward),
 * and the per-block attention of the ring step entered at decoder/ring.py:30-37.
 *
 * q   (B, Lq, Hq,  D)  strides sq_b, sq_l, sq_h   (head-axis slices of the packed
 * k,v (B, Lk, Hkv, D)  strides sk_*, sv_*          QKV buffer are accepted as is)
 * out (B, Lq, Hq,  D)  strides so_*
 * lse (B, Hq, Lq) fp32 contiguous, natural-log units; -inf for a query row that
 *                      sees no key (its out row is 0).
 * GQA: q head h reads kv head h / (Hq / Hkv).  causal != 0 masks key j for
 * query i when j > i + (Lk - Lq).  D in {64, 128}.  Every tensor: 16-byte aligned
 * pointer, strides that are multiples of 16 bytes (8 bf16 / 4 fp32 elements).
 * workspace: ody_attn_fwd_workspace_bytes(...) bytes, 256-byte aligned (the bf16
 * head_dim-128 kernel keeps a transposed copy of V and one int per 256-query block
 * there; 0 bytes = may be NULL).  For a call with too few 256-query blocks to fill the
 * chip (a ring step of few queries against a long key block) the size includes fp32
 * partial results: the kernel then cuts every block's key range into 2 or 4 parts and a
 * second kernel merges them by their log-sum-exp.  A workspace with room for the V copy
 * and the flags only is accepted too; such a call runs unsplit.
 */
size_t ody_attn_fwd_workspace_bytes(int B, int Lq, int Lk, int Hq, int Hkv, int D, int dtype);
int ody_attn_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                 int B, int Lq, int Lk, int Hq, int Hkv, int D,
                 int64_t sq_b, int64_t sq_l, int64_t sq_h,
                 int64_t sk_b, int64_t sk_l, int64_t sk_h,
                 int64_t sv_b, int64_t sv_l, int64_t sv_h,
                 int64_t so_b, int64_t so_l, int64_t so_h,
                 float scale, int causal, int dtype,
                 void* workspace, size_t workspace_bytes, void* stream);

/* ody_attn_fwd for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose
 * attention routine allocates through PyTorch.  Same arguments and results as ody_attn_fwd, without
 * the workspace: the scratch of the bf16 head_dim-128 kernel (transposed image of V, block flags,
 * the fp32 parts of a call that cuts its key range) lives in a buffer of
 * ODY_ATTN_FWD_NOALLOC_SCRATCH_BYTES that the library itself holds on every GPU it runs on, for
 * the life of the process.  Bit for bit the results of ody_attn_fwd with a workspace of the same
 * kind: a call whose fp32 parts do not fit the buffer runs unsplit (as ody_attn_fwd does with a
 * workspace without room for them).  The call allocates and frees nothing and synchronises
 * nothing; a shape whose V image and flags exceed the buffer (more than about 131000 key rows
 * over all kv heads and batches) returns ODY_ERR_WORKSPACE.
 * All calls on one GPU share that GPU's buffer: calls that may overlap there (different
 * streams, different threads) race, so keep them on one stream or order them with events.  The
 * first call on a device looks up the buffer's address; make that call outside graph capture.
 */
#define ODY_ATTN_FWD_NOALLOC_SCRATCH_BYTES ((32u << 20) + (64u << 10))
int ody_attn_fwd_noalloc(const void* q, const void* k, const void* v, void* out, float* lse,
                         int B, int Lq, int Lk, int Hq, int Hkv, int D,
                         int64_t sq_b, int64_t sq_l, int64_t sq_h,
                         int64_t sk_b, int64_t sk_l, int64_t sk_h,
                         int64_t sv_b, int64_t sv_l, int64_t sv_h,
                         int64_t so_b, int64_t so_l, int64_t so_h,
                         float scale, int causal, int dtype, void* stream);

/* Backward of the above (flash_attn's backward as run by autograd through
 * decoder/odysseus.py:256-263).  `out` and `lse` are the forward results -- or,
 * for a ring step, the FINAL merged out / lse, which is what makes the per-block
 * gradients sum to the gradient of the unsplit attention.
 * dq/dk/dv have the shapes of q/k/v with their own strides.  dK and dV of a kv
 * head are summed over its query-head group inside the kernel (deterministic,
 * no atomics).  `flags` is a sum of
 *   ODY_BWD_ACCUMULATE_DQ     the kernel adds into dq (in fp32, rounded once per call when dq is bf16);
 *   ODY_BWD_DQ_F32            dq is an fp32 buffer (strides in fp32 elements) although q is bf16: with
 *                             ACCUMULATE this is the ring step's running dq, exact over any number of key
 *                             blocks and rounded once by the caller at the end (ody_cast_from_f32);
 *   ODY_BWD_REUSE_QUERY_SIDE  q, out, lse, dout and the workspace are those of the previous call: delta and
 *                             the other query-side scratch in the workspace are taken as they are (the ring
 *                             step calls once per key block with the same queries);
 *   ODY_BWD_KEEP_DS           spends memory to save arithmetic (no counterpart in the reference): the dK/dV
 *                             kernel keeps dS, rounded to bf16 as it is used there, in the workspace, and dQ is
 *                             one product dS K over it instead of a second pass over S, dP and dS.  Same
 *                             results.  For bf16, head_dim 128, Lq and Lk multiples of 256 and, if causal,
 *                             Lq == Lk (ody_attn_bwd_ds_bytes(...) > 0); the workspace then holds
 *                             ody_attn_bwd_workspace_bytes(...) + ody_attn_bwd_ds_bytes(...) bytes, the latter
 *                             2 bytes per visible (query, key) pair: about B * Hq * Lq * Lk bytes when causal,
 *                             twice that for a full block.
 * workspace: ody_attn_bwd_workspace_bytes(...) bytes, 256-byte aligned (delta, and for
 * the bf16 head_dim-128 kernels transposed copies of K, Q and dO, plus fp32 partial dK / dV
 * or dQ where grouped-query attention, or a call with one short side, is cut into parts
 * that a second kernel adds up in a fixed order).
 */
enum ody_attn_bwd_flags { ODY_BWD_ACCUMULATE_DQ = 1, ODY_BWD_DQ_F32 = 2, ODY_BWD_REUSE_QUERY_SIDE = 4, ODY_BWD_KEEP_DS = 8 };
size_t ody_attn_bwd_workspace_bytes(int B, int Lq, int Lk, int Hq, int Hkv, int D, int dtype);
size_t ody_attn_bwd_ds_bytes(int B, int Lq, int Lk, int Hq, int Hkv, int D, int dtype, int causal);
int ody_attn_bwd(const void* q, const void* k, const void* v, const void* out, const float* lse,
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
                 void* workspace, size_t workspace_bytes, void* stream);

/* Online-softmax merge of one key block's partial result into the running one
 * (the update rule of ring_flash_attn, reached from decoder/ring.py:30-37):
 *   lse' = logaddexp(lse, lse_blk)
 *   out' = out * e^(lse - lse') + out_blk * e^(lse_blk - lse')
 * out_acc (B, L, H, D) fp32 contiguous, updated in place; lse_acc (B, H, L) fp32
 * updated in place; out_blk (B, L, H, D) of `dtype` with strides sb_*; lse_blk
 * (B, H, L) fp32.  A side whose lse is -inf contributes nothing.
 */
int ody_lse_merge(float* out_acc, float* lse_acc, const void* out_blk, const float* lse_blk,
                  int B, int L, int H, int D, int64_t sb_b, int64_t sb_l, int64_t sb_h,
                  int dtype, void* stream);

/* Rounds an fp32 array to `dtype` (n elements, both 16-byte aligned, n a multiple of 8): the last step of a
 * result that was accumulated in fp32 over the key blocks of a ring step (running out, running dq).
 */
int ody_cast_from_f32(const float* src, void* dst, int64_t n, int dtype, void* stream);

/* ---- dense linears ------------------------------------------------------
 * C (M, N) = op(A) * op(B), row-major, leading dimensions in elements.
 *   ODY_GEMM_NT  C = A (M,K) * B (N,K)^T   forward  X W^T   utils/linear_tpsp.py:173,
 *                                                           :588, utils/linear_zero3.py:44
 *   ODY_GEMM_NN  C = A (M,K) * B (K,N)     dgrad    dY W    utils/linear_tpsp.py:217,
 *                                                           utils/linear_zero3.py:68
 *   ODY_GEMM_TN  C = A (K,M)^T * B (K,N)   wgrad    dY^T X  utils/linear_tpsp.py:291,
 *                                                           utils/linear_zero3.py:74
 * bias (N) of `dtype` or NULL is added to every row (utils/linear_tpsp.py:175-176).
 * If accumulate != 0, C += result (C read in `dtype`, added in fp32).
 * bf16: A and B 16-byte aligned with lda, ldb, N and their contiguous extents multiples of 8, C and
 * bias 8-byte aligned with ldc a multiple of 4.  fp32: any shape and alignment.
 * workspace (optional, 16-byte aligned): with ody_gemm_workspace_bytes(...) > 0 bytes of it a product
 * with a long K and few output tiles (a weight gradient) is computed over several ranges of K at once
 * and summed in fp32; without it (NULL / too small) the same result comes from one pass over K.
 */
enum ody_gemm_op { ODY_GEMM_NT = 0, ODY_GEMM_NN = 1, ODY_GEMM_TN = 2 };
size_t ody_gemm_workspace_bytes(int op, int M, int N, int K, int dtype);
int ody_gemm(int op, const void* A, const void* B, void* C, const void* bias,
             int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
             int accumulate, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ---- linears fused with their elementwise neighbour -----------------------------
 * The same products as ody_gemm's NT / NN with the operation that follows them in the layer done in the
 * product's epilogue, so that the intermediate never makes a round trip through HBM.  Row-major, leading
 * dimensions in elements.  bf16 shapes made of whole 256 x 256 tiles with K a multiple of 64 and 16-byte
 * aligned rows take one fused kernel; everything else (fp32, ragged or small shapes) runs as the product
 * followed by the stand-alone kernel, with the same result.
 *
 * ody_linear_residual     y (M, N) = x (M, K) W (N, K)^T + residual (M, N): the output projection and the
 *                         down projection together with the decoder layer's residual add
 *                         (utils/linear_tpsp.py:588 / utils/linear_zero3.py:44, then decoder/ring.py:80,86).
 *                         The sum is formed in fp32 and rounded once.  y may be the residual buffer itself only
 *                         when the shape takes the unfused path; pass distinct buffers.
 * ody_linear_swiglu       gate_up (T, 2 I) = x (T, K) Wgu (2 I, K)^T and h (T, I) = silu(gate) * up
 *                         (decoder/odysseus.py:293-295); gate_up is kept because the backward needs it.
 * ody_linear_dgrad_swiglu d_gate_up (T, 2 I) = SwiGLU backward of (gate_up, dh) with dh = dy (T, K) Wd (K, I):
 *                         the input gradient of the down projection (utils/linear_zero3.py:68) feeding the
 *                         backward of decoder/odysseus.py:295; dh itself is never stored.  workspace:
 *                         ody_linear_dgrad_swiglu_workspace_bytes(...) bytes (0 when the shape takes the fused
 *                         kernel; otherwise room for dh), 16-byte aligned.  The query goes by the shape alone and
 *                         assumes 16-byte aligned pointers and leading dimensions that are multiples of 8: operands
 *                         without them take the two-kernel path whatever the shape and need T * I elements of
 *                         workspace (the call returns ODY_ERR_WORKSPACE and says so if it is missing).
 */
int ody_linear_residual(const void* x, const void* w, const void* residual, void* y, int M, int N, int K,
                        int64_t ldx, int64_t ldw, int64_t ld_res, int64_t ldy, int dtype, void* stream);
int ody_linear_swiglu(const void* x, const void* w_gate_up, void* gate_up, void* h, int T, int I, int K,
                      int64_t ldx, int64_t ldw, int64_t ld_gu, int64_t ld_h, int dtype, void* stream);
size_t ody_linear_dgrad_swiglu_workspace_bytes(int T, int I, int K, int dtype);
int ody_linear_dgrad_swiglu(const void* dy, const void* w_down, const void* gate_up, void* d_gate_up, int T, int I,
                            int K, int64_t ld_dy, int64_t ldw, int64_t ld_gu, int64_t ld_dgu, int dtype,
                            void* workspace, size_t workspace_bytes, void* stream);

/* ---- SwiGLU -------------------------------------------------------------
 * decoder/odysseus.py:293-295: a1, a3 = gate_up.chunk(2, -1); h = silu(a1) * a3.
 * gate_up (T, 2*I) row stride ld_gu; h (T, I) row stride ld_h.
 * bwd: d_gate_up (T, 2*I) from gate_up and dh.
 */
int ody_swiglu_fwd(const void* gate_up, void* h, int T, int I, int64_t ld_gu, int64_t ld_h,
                   int dtype, void* stream);
int ody_swiglu_bwd(const void* gate_up, const void* dh, void* d_gate_up, int T, int I,
                   int64_t ld_gu, int64_t ld_dh, int64_t ld_dgu, int dtype, void* stream);

/* ---- RMSNorm ------------------------------------------------------------
 * HF LlamaRMSNorm as called by the decoder layer (decoder/ring.py:67,84):
 * y = w * (x * rsqrt(mean(x^2) + eps)) with fp32 statistics.  x, y (T, d)
 * contiguous; rstd (T) fp32 is written by fwd and read by bwd.
 * bwd: dx (T, d); dw_partial (n_partial, d) fp32 partial column sums, where
 * n_partial = ody_rmsnorm_bwd_partials(T); the caller (or ody_rmsnorm_bwd with
 * dw != NULL) reduces them: dw (d) of `dtype`.  dx_add (T, d) of `dtype` or NULL is
 * added to dx in fp32 before the one rounding: the gradient that reaches the
 * norm's input over the residual connection (decoder/ring.py:80,86), so that the
 * sum of the two branches costs no pass of its own.  d at most 8192 (bf16) /
 * 4096 (fp32): larger rows return ODY_ERR_UNSUPPORTED.
 */
int ody_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd, int T, int d, float eps,
                    int dtype, void* stream);
int ody_rmsnorm_bwd_partials(int T);
int ody_rmsnorm_bwd(const void* x, const void* w, const float* rstd, const void* dy, const void* dx_add, void* dx,
                    float* dw_partial, void* dw, int T, int d, int dtype, void* stream);

/* ---- RoPE ---------------------------------------------------------------
 * HF rotary_emb + apply_rotary_pos_emb at decoder/odysseus.py:210-213
 * (half-rotation convention; angles computed in fp32 from position * base^(-2j/D),
 * cos/sin rounded to `dtype` before use, as HF does).
 * x (B, L, H, D) with strides sx_*, rotated IN PLACE for the first n_rot heads on
 * the head axis (q and k heads of the packed buffer are adjacent, v is left alone).
 * position_ids (B, L) int64 or NULL for arange(L).  inv_freq (D/2) fp32 is the
 * frequency table base^(-2j/D) as the caller's rotary module holds it (passing
 * the table keeps the angles bit-identical to the host's and admits scaled
 * variants); NULL evaluates base^(-2j/D) in the kernel.  inverse != 0 rotates by
 * the opposite angle (the backward pass).
 */
int ody_rope(void* x, const int64_t* position_ids, const float* inv_freq, int B, int L, int n_rot,
             int D, int64_t sx_b, int64_t sx_l, int64_t sx_h, float base, int inverse,
             int dtype, void* stream);

/* The same rotary embedding fused into its neighbours (bf16, head_dim 128), so that no pass over the packed
 * projection is left: the rotation of q and k (decoder/odysseus.py:210-213) rides in the epilogue of the QKV
 * projection (utils/linear_tpsp.py:173), and its backward in the epilogues of the attention backward.
 *
 * ody_rope_table   table (rows, D) bf16: table[r][2 j] = cos, table[r][2 j + 1] = sin of position_ids[r] *
 *                  inv_freq[j], j < D / 2 (NULL position_ids: r; NULL inv_freq: base^(-2j/D)), rounded to bf16 as
 *                  ody_rope rounds them.  rows = B * L in the order of the projection's rows; contiguous (ld_table = D).
 * ody_linear_rope  y (M, N) = x (M, K) w (N, K)^T with the first n_rot heads of D columns rotated by the table's row m
 *                  before the one rounding to bf16 (ody_gemm + ody_rope round twice).  Any shape: products the fused
 *                  kernel does not take run as the plain product followed by the rotation from the table.
 * ody_attn_bwd_rope  ody_attn_bwd whose dq and dk leave the kernels rotated back by the negative angle, i.e. as the
 *                  gradient of the projection before its rotary embedding: rope_table_q holds the rows of the
 *                  queries (B * Lq, pitch D), rope_table_k those of the keys (B * Lk).  Not with ODY_BWD_ACCUMULATE_DQ
 *                  or ODY_BWD_DQ_F32.
 */
int ody_rope_table(const int64_t* position_ids, const float* inv_freq, int64_t rows, int D, float base,
                   void* table, void* stream);
int ody_linear_rope(const void* x, const void* w, const void* table, void* y, int M, int N, int K, int n_rot,
                    int D, int64_t ldx, int64_t ldw, int64_t ld_table, int64_t ldy, int dtype, void* stream);
int ody_attn_bwd_rope(const void* q, const void* k, const void* v, const void* out, const float* lse,
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
                      const void* rope_table_q, const void* rope_table_k);

/* ---- attention dropout ------------------------------------------------------
 * The dropout_p argument of the attention routine the reference calls (decoder/odysseus.py:228, 256-263; it
 * passes config.attention_dropout while training, 0.0 in its own configurations).  ody_attn_fwd / ody_attn_bwd with
 * two more arguments: an entry of the softmax matrix P is dropped with probability p_drop before P . V and the
 * kept entries are scaled by 1 / (1 - p_drop); lse is that of the full P.  Which entries are dropped is a fixed
 * function of (seed, batch, query head, query, key) -- a 32-bit counter hash, restated on the host in
 * oracle/odysseus_oracle.py -- so the backward reproduces the forward's mask from the same seed.  The reference's
 * routine draws its mask from a Philox stream of its own: masks differ, the distribution and the arithmetic given a
 * mask are the same.  bf16 and fp32, head_dim 64 or 128; bf16 on the library's plain kernels (no key split, no kept dS,
 * no rotary tables: ODY_BWD_KEEP_DS is refused); p_drop = 0 is exactly ody_attn_fwd / ody_attn_bwd.  Workspaces as
 * for those.
 */
int ody_attn_fwd_dropout(const void* q, const void* k, const void* v, void* out, float* lse,
                         int B, int Lq, int Lk, int Hq, int Hkv, int D,
                         int64_t sq_b, int64_t sq_l, int64_t sq_h,
                         int64_t sk_b, int64_t sk_l, int64_t sk_h,
                         int64_t sv_b, int64_t sv_l, int64_t sv_h,
                         int64_t so_b, int64_t so_l, int64_t so_h,
                         float scale, int causal, int dtype,
                         void* workspace, size_t workspace_bytes, void* stream, float p_drop, uint64_t seed);
int ody_attn_bwd_dropout(const void* q, const void* k, const void* v, const void* out, const float* lse,
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
                         void* workspace, size_t workspace_bytes, void* stream, float p_drop, uint64_t seed);

/* ---- optimizer ------------------------------------------------------------
 * One step of torch.optim.AdamW (the optimizer of the reference's training loop, train.py:170,216) on one
 * tensor of n elements, in one pass instead of the host framework's seven element-wise passes:
 *   p *= 1 - lr * weight_decay;  m = beta1 m + (1 - beta1) g;  v = beta2 v + (1 - beta2) g^2;
 *   p -= lr / (1 - beta1^step) * m / (sqrt(v) / sqrt(1 - beta2^step) + eps)
 * param, grad, exp_avg, exp_avg_sq: contiguous arrays of `dtype`, 16-byte aligned; fp32 arithmetic, one rounding per
 * stored value.  step counts from 1.
 */
int ody_adamw(void* param, const void* grad, void* exp_avg, void* exp_avg_sq, int64_t n, float lr, float beta1,
              float beta2, float eps, float weight_decay, int64_t step, int dtype, void* stream);

/* ---- cross-entropy over the vocabulary --------------------------------------
 * flash_attn.losses.cross_entropy.CrossEntropyLoss(inplace_backward=True) as the training loop
 * uses it (train.py:8,173,212-214): softmax cross-entropy of logits (T, V) (row stride ld,
 * `dtype`) against labels (T) int64, statistics in fp32.
 * fwd: lse (T) = log sum_v exp(logits[t, v]); losses (T) = lse[t] - logits[t, labels[t]], and 0
 *      for a token whose label is ignore_index (or outside [0, V): such a token is skipped, never
 *      dereferenced).  If reduced != NULL: reduced[0] = mean of the losses over the counted
 *      tokens, reduced[1] = their number (one block, fixed order: deterministic).
 * bwd: overwrites logits IN PLACE with d loss / d logits = (softmax - onehot(label)) * g, where
 *      g = dloss[t] if dloss != NULL (per-token upstream gradient), else grad_loss[0] / reduced[1]
 *      (mean reduction; grad_loss is a DEVICE scalar, so nothing synchronises).  Rows of skipped
 *      tokens become 0.
 * 16-byte accesses are used when logits is 16-byte aligned and ld a multiple of 8 (bf16) / 4 (fp32).
 */
int ody_cross_entropy_fwd(const void* logits, const int64_t* labels, float* losses, float* lse, float* reduced,
                          int T, int V, int64_t ld, int64_t ignore_index, int dtype, void* stream);
int ody_cross_entropy_bwd(void* logits, const int64_t* labels, const float* lse, const float* reduced,
                          const float* grad_loss, const float* dloss, int T, int V, int64_t ld,
                          int64_t ignore_index, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ODYSSEUS_HIP_H */
