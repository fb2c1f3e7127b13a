"""CPU oracle for the per-rank compute of the Odysseus decoder layer.

THIS FILE IS TEST INFRASTRUCTURE.  It is a plain-PyTorch (CPU, fp32 or fp64)
restatement of the arithmetic that the reference performs on one rank at
world_size = 1.  Only the test-suite, the smoke check and the CPU-baseline leg
of the benchmark may import it; the product package never does.

The reference holds none of this arithmetic itself: it calls flash_attn, HF
transformers (RoPE, RMSNorm, SiLU) and torch.matmul.  Each function below
therefore cites the reference *call site* that fixes the semantics (layout,
order of operations, which slice is which) and restates the published formula
of the third-party routine.

How each function is pinned (tests/test_oracle.py):

  rmsnorm            closed form vs. an independent fp64 formula; scale
                     invariance rms(a*x) == rms(x) as eps -> 0
  rope_cos_sin,      position 0 is the identity; pairwise norm preserved;
  apply_rope         <rope(q,m), rope(k,n)> depends only on m-n; equals the
                     installed transformers' apply_rotary_pos_emb
  attention_fwd      == torch.nn.functional.scaled_dot_product_attention
                     (causal, enable_gqa) and brute-force softmax on tiny
                     inputs; lse == torch.logsumexp of the masked scores;
                     row 0: out == v[0], lse == q0.k0*scale
  attention_bwd      == torch.autograd through the brute-force softmax (fp64);
                     sum_d dO*O == sum_j P*dP; GQA == MHA on repeated K/V with
                     dK/dV summed per group
  lse_merge,         merging per-block (out, lse) over a partition of the keys
  ring_attention_*   == unsplit attention over the concatenated keys, forward
                     and all gradients; merge with lse = -inf is the identity
  linear_*           == torch.nn.functional.linear + autograd in fp64
  swiglu_mlp_*       == silu(x Wg^T) * (x Wu^T) then Wd, the HF LlamaMLP
                     formula with gate = W[:i], up = W[i:]
  cross_entropy_*    == torch.nn.functional.cross_entropy (mean, ignore_index) and its
                     autograd gradient in fp64; rows of the gradient sum to zero
  adamw_step         == torch.optim.AdamW over several steps in fp64 (parameter and
                     both moments); with zero gradient only the weight decay acts
  attention_block,   autograd of the composed functions vs. the explicit
  decoder_layer_*    backward formulas in this file
  dropout (the       given a mask: attention_fwd / attention_bwd == autograd through the brute-force softmax with
  dropout_p, seed    the same mask applied as torch.nn.functional.dropout does (fp64); p = 0 is the undropped
  arguments)         result; the kept fraction of dropout_keep_mask is 1 - p within sampling error, and it is the
                     same for every way of slicing the index ranges.  The mask ITSELF (dropout_keep_mask) is this
                     build's own counter hash: the reference's routine draws from flash-attn's Philox stream, which
                     nothing here can reproduce -- the mask's bit pattern is parity-unpinned, its distribution and
                     the arithmetic are not

Parity unpinned (nothing in the reference, its tests, or mathematics fixes it):
the exact bf16 rounding sequence of flash-attn's CUDA kernels (P rounded to
bf16 before P.V, dS rounding) -- covered by the 2e-2 tolerance against this
fp32 oracle.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch

NEG_INF = float("-inf")


# --------------------------------------------------------------------------
# RMSNorm  (caller side of the hot path: decoder/ring.py:67,84 call
# input_layernorm / post_attention_layernorm, HF LlamaRMSNorm)
# --------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """w * (x * rsqrt(mean(x^2) + eps)), statistics in fp32 at least."""
    ct = torch.float64 if x.dtype == torch.float64 else torch.float32
    xf = x.to(ct)
    var = xf.pow(2).mean(-1, keepdim=True)
    y = xf * torch.rsqrt(var + eps)
    return weight * y.to(x.dtype)


def rmsnorm_bwd(x: torch.Tensor, weight: torch.Tensor, dy: torch.Tensor, eps: float = 1e-6):
    """Explicit gradient of rmsnorm: returns (dx, dweight)."""
    ct = torch.float64 if x.dtype == torch.float64 else torch.float32
    xf, wf, dyf = x.to(ct), weight.to(ct), dy.to(ct)
    d = x.shape[-1]
    rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    xhat = xf * rstd
    g = dyf * wf
    dx = rstd * (g - xhat * (g * xhat).sum(-1, keepdim=True) / d)
    dw = (dyf * xhat).reshape(-1, d).sum(0)
    return dx.to(x.dtype), dw.to(weight.dtype)


# --------------------------------------------------------------------------
# RoPE  (decoder/odysseus.py:210-213: rotary_emb(value_states, position_ids)
# then apply_rotary_pos_emb(q, k, cos, sin); HF half-rotation convention)
# --------------------------------------------------------------------------
def rope_cos_sin(position_ids: torch.Tensor, head_dim: int, base: float = 10000.0,
                 dtype: torch.dtype = torch.float32) -> Tuple[torch.Tensor, torch.Tensor]:
    """position_ids (B, L) -> cos, sin (B, L, D); angles in fp32 then cast."""
    ct = torch.float64 if dtype == torch.float64 else torch.float32
    j = torch.arange(0, head_dim, 2, dtype=torch.int64).to(ct)
    inv_freq = 1.0 / (base ** (j / head_dim))                       # (D/2,)
    theta = position_ids.to(ct)[..., None] * inv_freq               # (B, L, D/2)
    emb = torch.cat((theta, theta), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def _rotate_half(x: torch.Tensor) -> torch.Tensor:
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x (B, L, H, D); cos/sin (B, L, D).  x*cos + rotate_half(x)*sin."""
    c, s = cos[:, :, None, :], sin[:, :, None, :]
    return x * c + _rotate_half(x) * s


def apply_rope_bwd(dy: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Gradient of apply_rope w.r.t. x: rotation by the opposite angle."""
    c, s = cos[:, :, None, :], sin[:, :, None, :]
    h = dy.shape[-1] // 2
    t = dy * s
    return dy * c + torch.cat((t[..., h:], -t[..., :h]), dim=-1)


# --------------------------------------------------------------------------
# Attention  (decoder/odysseus.py:256-263 -> HF _flash_attention_forward ->
# flash_attn_func(q, k, v, dropout_p=0, softmax_scale=None, causal=True);
# layout (B, L, H, D); GQA: q head h reads kv head h // (Hq / Hkv))
# --------------------------------------------------------------------------
def _ct(t: torch.Tensor) -> torch.dtype:
    return torch.float64 if t.dtype == torch.float64 else torch.float32


_M32 = 0xFFFFFFFF


def _mix32(x: torch.Tensor) -> torch.Tensor:
    """The 32-bit finalizer of MurmurHash3 on int64 tensors holding unsigned 32-bit values."""
    x = x ^ (x >> 16)
    x = (x * 0x85EBCA6B) & _M32
    x = x ^ (x >> 13)
    x = (x * 0xC2B2AE35) & _M32
    return x ^ (x >> 16)


def dropout_keep_mask(seed: int, p_drop: float, B: int, Hq: int, q_idx: torch.Tensor, k_idx: torch.Tensor) -> torch.Tensor:
    """Which entries of P survive dropout: bool (B, Hq, len(q_idx), len(k_idx)).  The decision for (b, h, q, k) is a
    fixed function of the seed and the four indices (a counter hash: no state, any kernel can evaluate any entry):
        u = mix(seed32 ^ (b * Hq + h) * 0x85ebca77);  r = mix(u + q * 0x9e3779b1);  x = mix(r ^ k * 0xc2b2ae3d)
    kept iff x >= p_drop * 2^32 (all in unsigned 32-bit arithmetic; seed32 = low word ^ high word of the seed)."""
    seed &= 0xFFFFFFFFFFFFFFFF
    seed32 = (seed ^ (seed >> 32)) & _M32
    t = p_drop * 4294967296.0
    thresh = 4294967295 if t >= 4294967295.0 else (1 if t < 1.0 else int(t))
    bh = torch.arange(B * Hq, dtype=torch.int64).view(B, Hq, 1, 1)
    u = _mix32(seed32 ^ ((bh * 0x85EBCA77) & _M32))
    r = _mix32((u + ((q_idx.to(torch.int64).view(1, 1, -1, 1) * 0x9E3779B1) & _M32)) & _M32)
    x = _mix32(r ^ ((k_idx.to(torch.int64).view(1, 1, 1, -1) * 0xC2B2AE3D) & _M32))
    return x >= thresh


def attention_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, causal: bool = True,
                  scale: Optional[float] = None, block: int = 1024, dropout_p: float = 0.0,
                  seed: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    """q (B, Lq, Hq, D), k/v (B, Lk, Hkv, D) -> out (B, Lq, Hq, D), lse (B, Hq, Lq).

    dropout_p > 0 (the dropout_p of the routine called at decoder/odysseus.py:256-263): entries of P are dropped
    per dropout_keep_mask and the kept ones scaled by 1 / (1 - dropout_p) before P . V; lse is that of the full P.

    Causal masking is aligned to the bottom-right corner (key j visible to
    query i iff j <= i + Lk - Lq), which for Lq == Lk is j <= i.  Computed one
    block of query rows at a time so that L = 32K fits in host memory.
    """
    B, Lq, Hq, D = q.shape
    Lk, Hkv = k.shape[1], k.shape[2]
    assert Hq % Hkv == 0
    G = Hq // Hkv
    ct = _ct(q)
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    qh = q.to(ct).permute(0, 2, 1, 3)                                   # (B, Hq, Lq, D)
    kh = k.to(ct).permute(0, 2, 1, 3).repeat_interleave(G, dim=1)       # (B, Hq, Lk, D)
    vh = v.to(ct).permute(0, 2, 1, 3).repeat_interleave(G, dim=1)
    out = torch.empty(B, Hq, Lq, D, dtype=ct)
    lse = torch.empty(B, Hq, Lq, dtype=ct)
    off = Lk - Lq
    for i0 in range(0, Lq, block):
        i1 = min(i0 + block, Lq)
        kend = min(Lk, i1 + off) if causal else Lk
        kend = max(kend, 0)
        s = torch.matmul(qh[:, :, i0:i1], kh[:, :, :kend].transpose(-1, -2)) * scale
        if causal:
            ii = torch.arange(i0, i1)[:, None] + off
            jj = torch.arange(kend)[None, :]
            s = s.masked_fill(jj > ii, NEG_INF)
        l = torch.logsumexp(s, dim=-1)                                  # -inf for empty rows
        p = torch.exp(s - torch.where(torch.isinf(l), torch.zeros_like(l), l)[..., None])
        if dropout_p > 0.0:
            keep = dropout_keep_mask(seed, dropout_p, B, Hq, torch.arange(i0, i1), torch.arange(kend))
            p = torch.where(keep, p / (1.0 - dropout_p), torch.zeros_like(p))
        out[:, :, i0:i1] = torch.matmul(p, vh[:, :, :kend])
        lse[:, :, i0:i1] = l
    return out.permute(0, 2, 1, 3).contiguous().to(q.dtype), lse


def attention_bwd(q, k, v, out, lse, dout, causal: bool = True, scale: Optional[float] = None,
                  block: int = 1024, dropout_p: float = 0.0, seed: int = 0):
    """Explicit flash-attention backward: returns (dq, dk, dv).  With dropout (mask M, scale c = 1 / (1 - p)):
    dV = (c M P)^T dO, dP = c M (dO V^T), and delta, dS, dQ, dK as below.

    P = exp(S - lse), dV = P^T dO, dP = dO V^T, delta_i = sum_d dO_id O_id,
    dS = P * (dP - delta), dQ = dS K * scale, dK = dS^T Q * scale; dK and dV of
    a kv head are summed over the q heads of its group.  `out` and `lse` may be
    the result of a wider softmax than (k, v) alone: that is how the ring step
    uses it (final lse / final out for every key block).
    """
    B, Lq, Hq, D = q.shape
    Lk, Hkv = k.shape[1], k.shape[2]
    G = Hq // Hkv
    ct = _ct(q)
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    qh = q.to(ct).permute(0, 2, 1, 3)
    kh = k.to(ct).permute(0, 2, 1, 3).repeat_interleave(G, dim=1)
    vh = v.to(ct).permute(0, 2, 1, 3).repeat_interleave(G, dim=1)
    oh = out.to(ct).permute(0, 2, 1, 3)
    doh = dout.to(ct).permute(0, 2, 1, 3)
    lse = lse.to(ct)
    delta = (oh * doh).sum(-1)                                          # (B, Hq, Lq)
    dq = torch.zeros_like(qh)
    dk = torch.zeros_like(kh)
    dv = torch.zeros_like(vh)
    off = Lk - Lq
    for i0 in range(0, Lq, block):
        i1 = min(i0 + block, Lq)
        kend = max(min(Lk, i1 + off) if causal else Lk, 0)
        s = torch.matmul(qh[:, :, i0:i1], kh[:, :, :kend].transpose(-1, -2)) * scale
        if causal:
            ii = torch.arange(i0, i1)[:, None] + off
            jj = torch.arange(kend)[None, :]
            s = s.masked_fill(jj > ii, NEG_INF)
        l = lse[:, :, i0:i1]
        p = torch.exp(s - torch.where(torch.isinf(l), torch.zeros_like(l), l)[..., None])
        dp = torch.matmul(doh[:, :, i0:i1], vh[:, :, :kend].transpose(-1, -2))
        pd = p
        if dropout_p > 0.0:
            keep = dropout_keep_mask(seed, dropout_p, B, Hq, torch.arange(i0, i1), torch.arange(kend))
            pd = torch.where(keep, p / (1.0 - dropout_p), torch.zeros_like(p))
            dp = torch.where(keep, dp / (1.0 - dropout_p), torch.zeros_like(dp))
        dv[:, :, :kend] += torch.matmul(pd.transpose(-1, -2), doh[:, :, i0:i1])
        ds = p * (dp - delta[:, :, i0:i1, None])
        dq[:, :, i0:i1] = torch.matmul(ds, kh[:, :, :kend]) * scale
        dk[:, :, :kend] += torch.matmul(ds.transpose(-1, -2), qh[:, :, i0:i1]) * scale
    dk = dk.view(B, Hkv, G, Lk, D).sum(2)
    dv = dv.view(B, Hkv, G, Lk, D).sum(2)
    f = lambda t: t.permute(0, 2, 1, 3).contiguous().to(q.dtype)
    return f(dq), f(dk), f(dv)


def attention_naive(q, k, v, causal: bool = True, scale: Optional[float] = None, keep: Optional[torch.Tensor] = None,
                    dropout_p: float = 0.0):
    """Differentiable brute force (materialises the scores); small inputs only.  keep: a bool mask (B, Hq, Lq, Lk) of
    the entries of P that survive dropout, scaled by 1 / (1 - dropout_p)."""
    B, Lq, Hq, D = q.shape
    Lk, Hkv = k.shape[1], k.shape[2]
    G = Hq // Hkv
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    qh = q.permute(0, 2, 1, 3)
    kh = k.permute(0, 2, 1, 3).repeat_interleave(G, dim=1)
    vh = v.permute(0, 2, 1, 3).repeat_interleave(G, dim=1)
    s = torch.matmul(qh, kh.transpose(-1, -2)) * scale
    if causal:
        ii = torch.arange(Lq)[:, None] + (Lk - Lq)
        jj = torch.arange(Lk)[None, :]
        s = s.masked_fill(jj > ii, NEG_INF)
    lse = torch.logsumexp(s, dim=-1)
    p = torch.softmax(s, dim=-1)
    if keep is not None:
        p = torch.where(keep, p / (1.0 - dropout_p), torch.zeros_like(p))
    return torch.matmul(p, vh).permute(0, 2, 1, 3), lse


# --------------------------------------------------------------------------
# Ring step: block attention + online-softmax merge  (entered at
# decoder/ring.py:30-37 -> ring_flash_attn; that package is not vendored and
# unpinned, its published update rule is restated here)
# --------------------------------------------------------------------------
def lse_merge(out: torch.Tensor, lse: torch.Tensor, out_blk: torch.Tensor, lse_blk: torch.Tensor):
    """Fold one block's (out_blk, lse_blk) into the running (out, lse).

    out (B, L, H, D) fp32 running accumulator, lse (B, H, L);
    lse' = logaddexp(lse, lse_blk); out' = out*e^(lse-lse') + out_blk*e^(lse_blk-lse').
    A side whose lse is -inf contributes nothing.
    """
    ct = _ct(out)
    new = torch.logaddexp(lse.to(ct), lse_blk.to(ct))
    safe = torch.where(torch.isinf(new), torch.zeros_like(new), new)
    wa = torch.exp(lse.to(ct) - safe).permute(0, 2, 1)[..., None]       # (B, L, H, 1)
    wb = torch.exp(lse_blk.to(ct) - safe).permute(0, 2, 1)[..., None]
    return out.to(ct) * wa + out_blk.to(ct) * wb, new


def ring_attention_fwd(q, k_blocks: Sequence[torch.Tensor], v_blocks: Sequence[torch.Tensor],
                       causal_block: Optional[int] = 0, scale: Optional[float] = None):
    """Q against a list of KV blocks; block `causal_block` is the causal diagonal."""
    B, Lq, Hq, D = q.shape
    ct = _ct(q)
    out = torch.zeros(B, Lq, Hq, D, dtype=ct)
    lse = torch.full((B, Hq, Lq), NEG_INF, dtype=ct)
    for b, (kb, vb) in enumerate(zip(k_blocks, v_blocks)):
        ob, lb = attention_fwd(q, kb, vb, causal=(b == causal_block), scale=scale)
        out, lse = lse_merge(out, lse, ob, lb)
    return out.to(q.dtype), lse


def ring_attention_bwd(q, k_blocks, v_blocks, out, lse, dout, causal_block: Optional[int] = 0,
                       scale: Optional[float] = None):
    """Per block flash backward with the FINAL lse/out; dQ summed over blocks."""
    ct = _ct(q)
    dq = torch.zeros_like(q, dtype=ct)
    dks, dvs = [], []
    for b, (kb, vb) in enumerate(zip(k_blocks, v_blocks)):
        dqb, dkb, dvb = attention_bwd(q, kb, vb, out, lse, dout, causal=(b == causal_block), scale=scale)
        dq += dqb.to(ct)
        dks.append(dkb)
        dvs.append(dvb)
    return dq.to(q.dtype), dks, dvs


# --------------------------------------------------------------------------
# Linears  (utils/linear_tpsp.py:173 fwd, :217 dgrad, :291 wgrad;
# utils/linear_zero3.py:44,68,74; utils/comm.py:10-19 flatten rule)
# --------------------------------------------------------------------------
def linear_fwd(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    y = torch.matmul(x, w.t())
    return y if b is None else y + b


def linear_bwd(x: torch.Tensor, w: torch.Tensor, dy: torch.Tensor, has_bias: bool = False):
    dx = torch.matmul(dy, w)
    dy2 = dy.reshape(-1, dy.shape[-1])
    x2 = x.reshape(-1, x.shape[-1])
    dw = torch.matmul(dy2.t(), x2)
    db = dy2.sum(0) if has_bias else None
    return dx, dw, db


# --------------------------------------------------------------------------
# SwiGLU MLP  (decoder/odysseus.py:293-295: a1, a3 = gate_up(x).chunk(2, -1);
# down(silu(a1) * a3))
# --------------------------------------------------------------------------
def swiglu(gu: torch.Tensor) -> torch.Tensor:
    a1, a3 = gu.chunk(2, dim=-1)
    return torch.nn.functional.silu(a1) * a3


def swiglu_bwd(gu: torch.Tensor, dh: torch.Tensor) -> torch.Tensor:
    a1, a3 = gu.chunk(2, dim=-1)
    sig = torch.sigmoid(a1)
    da1 = dh * a3 * sig * (1 + a1 * (1 - sig))
    da3 = dh * a1 * sig
    return torch.cat((da1, da3), dim=-1)


def swiglu_mlp_fwd(x, w_gate_up, w_down):
    return linear_fwd(swiglu(linear_fwd(x, w_gate_up)), w_down)


def swiglu_mlp_bwd(x, w_gate_up, w_down, dy):
    gu = linear_fwd(x, w_gate_up)
    h = swiglu(gu)
    dh, dwd, _ = linear_bwd(h, w_down, dy)
    dgu = swiglu_bwd(gu, dh)
    dx, dwgu, _ = linear_bwd(x, w_gate_up, dgu)
    return dx, dwgu, dwd


# --------------------------------------------------------------------------
# Cross-entropy  (train.py:173,212-214: flash_attn's CrossEntropyLoss on logits (T, V) and
# labels (T); mean over the tokens whose label is not ignore_index)
# --------------------------------------------------------------------------
def cross_entropy_fwd_bwd(logits: torch.Tensor, labels: torch.Tensor, ignore_index: int = -100,
                          grad_loss: float = 1.0):
    """Returns (mean loss, per-token losses, lse, d mean-loss / d logits * grad_loss)."""
    ct = _ct(logits)
    x = logits.to(ct)
    lse = torch.logsumexp(x, dim=-1)
    valid = labels != ignore_index
    safe = torch.where(valid, labels, torch.zeros_like(labels))
    losses = torch.where(valid, lse - x.gather(1, safe[:, None])[:, 0], torch.zeros_like(lse))
    n = valid.sum().clamp_min(1).to(ct)
    p = torch.exp(x - lse[:, None])
    onehot = torch.zeros_like(p).scatter_(1, safe[:, None], 1.0)
    dlogits = (p - onehot) * valid[:, None].to(ct) * (grad_loss / n)
    return losses.sum() / n, losses, lse, dlogits


# --------------------------------------------------------------------------
# AdamW  (train.py:170,216: torch.optim.AdamW with default betas, eps and weight decay)
# --------------------------------------------------------------------------
def adamw_step(param, grad, exp_avg, exp_avg_sq, step: int, lr: float, betas=(0.9, 0.999), eps: float = 1e-8,
               weight_decay: float = 1e-2):
    """One decoupled-weight-decay Adam step (Loshchilov & Hutter), as torch.optim.AdamW orders it.
    Returns the new (param, exp_avg, exp_avg_sq) in the compute dtype."""
    ct = _ct(param)
    p, g, m, v = (t.to(ct) for t in (param, grad, exp_avg, exp_avg_sq))
    b1, b2 = betas
    p = p * (1.0 - lr * weight_decay)
    m = b1 * m + (1.0 - b1) * g
    v = b2 * v + (1.0 - b2) * g * g
    bc1, bc2 = 1.0 - b1 ** step, 1.0 - b2 ** step
    p = p - (lr / bc1) * m / (v.sqrt() / (bc2 ** 0.5) + eps)
    return p, m, v


# --------------------------------------------------------------------------
# Attention block and decoder layer at world_size = 1
# (decoder/odysseus.py:170-271; layer wiring decoder/ring.py:65-86)
# --------------------------------------------------------------------------
def split_qkv(qkv: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int):
    """Packed projection (B, L, (Hq+2Hkv)*D) -> q, k, v head-axis slices in that order
    (decoder/odysseus.py:180-189)."""
    B, L, _ = qkv.shape
    t = qkv.view(B, L, n_heads + 2 * n_kv_heads, head_dim)
    return t[:, :, :n_heads], t[:, :, n_heads:n_heads + n_kv_heads], t[:, :, n_heads + n_kv_heads:]


def attention_block(x, w_qkv, w_o, n_heads, n_kv_heads, head_dim, position_ids=None,
                    rope_base: float = 10000.0, differentiable: bool = False):
    """x (1, L, d) -> (1, L, d).  Returns (y, lse)."""
    B, L, _ = x.shape
    assert B == 1, f"bsz: {B}"
    if position_ids is None:
        position_ids = torch.arange(L)[None]
    q, k, v = split_qkv(linear_fwd(x, w_qkv), n_heads, n_kv_heads, head_dim)
    cos, sin = rope_cos_sin(position_ids, head_dim, rope_base, x.dtype)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    if differentiable:
        o, lse = attention_naive(q, k, v, causal=True)
    else:
        o, lse = attention_fwd(q, k, v, causal=True)
    return linear_fwd(o.reshape(B, L, n_heads * head_dim), w_o), lse


def decoder_layer_fwd(x, p: dict, n_heads, n_kv_heads, head_dim, eps: float = 1e-6,
                      rope_base: float = 10000.0, position_ids=None, differentiable: bool = False):
    """p: ln1, w_qkv, w_o, ln2, w_gate_up, w_down.  h = x + attn(rms(x)); y = h + mlp(rms(h))."""
    a, _ = attention_block(rmsnorm(x, p["ln1"], eps), p["w_qkv"], p["w_o"], n_heads, n_kv_heads,
                           head_dim, position_ids, rope_base, differentiable)
    h = x + a
    return h + swiglu_mlp_fwd(rmsnorm(h, p["ln2"], eps), p["w_gate_up"], p["w_down"])


def decoder_layer_fwd_bwd(x, p: dict, dy, n_heads, n_kv_heads, head_dim, eps: float = 1e-6,
                          rope_base: float = 10000.0, position_ids=None):
    """Forward and explicit backward (blockwise attention, no autograd).

    Returns y and a dict of gradients keyed like `p` plus "x"."""
    B, L, d = x.shape
    if position_ids is None:
        position_ids = torch.arange(L)[None]
    # ---- forward, keeping what backward needs
    n1 = rmsnorm(x, p["ln1"], eps)
    qkv = linear_fwd(n1, p["w_qkv"])
    q0, k0, v = split_qkv(qkv, n_heads, n_kv_heads, head_dim)
    cos, sin = rope_cos_sin(position_ids, head_dim, rope_base, x.dtype)
    q, k = apply_rope(q0, cos, sin), apply_rope(k0, cos, sin)
    o, lse = attention_fwd(q, k, v, causal=True)
    o2 = o.reshape(B, L, n_heads * head_dim)
    h = x + linear_fwd(o2, p["w_o"])
    n2 = rmsnorm(h, p["ln2"], eps)
    y = h + swiglu_mlp_fwd(n2, p["w_gate_up"], p["w_down"])
    # ---- backward
    g = {}
    dn2, g["w_gate_up"], g["w_down"] = swiglu_mlp_bwd(n2, p["w_gate_up"], p["w_down"], dy)
    dh_n, g["ln2"] = rmsnorm_bwd(h, p["ln2"], dn2, eps)
    dh = dy + dh_n
    do2, g["w_o"], _ = linear_bwd(o2, p["w_o"], dh)
    dq, dk, dv = attention_bwd(q, k, v, o, lse, do2.view(B, L, n_heads, head_dim), causal=True)
    dq0, dk0 = apply_rope_bwd(dq, cos, sin), apply_rope_bwd(dk, cos, sin)
    dqkv = torch.cat((dq0, dk0, dv), dim=2).reshape(B, L, -1)
    dn1, g["w_qkv"], _ = linear_bwd(n1, p["w_qkv"], dqkv)
    dx_n, g["ln1"] = rmsnorm_bwd(x, p["ln1"], dn1, eps)
    g["x"] = dh + dx_n
    return y, g
