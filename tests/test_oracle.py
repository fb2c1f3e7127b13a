"""Pins the CPU oracle: every function is checked against a library routine, a closed
form, brute force on small inputs or an invariant -- chosen so that a dropped term,
a wrong sign or index, or a transposed operand fails at least one check.  (The
reference ships no golden vectors for this path; its own tests are differential.)"""
import math

import pytest
import torch
import torch.nn.functional as F

from conftest import randn
import odysseus_oracle as oracle

D64 = torch.float64


def r64(shape, seed, std=1.0):
    return randn(shape, seed, std).to(D64)


# ------------------------------------------------------------------ RMSNorm
def test_rmsnorm_closed_form_and_scale_invariance():
    x, w = r64((2, 5, 32), 1), r64((32,), 2)
    y = oracle.rmsnorm(x, w, 1e-6)
    ref = w * x / torch.sqrt((x * x).sum(-1, keepdim=True) / 32 + 1e-6)
    assert torch.allclose(y, ref, atol=1e-12)
    assert torch.allclose(oracle.rmsnorm(3.7 * x, w, 0.0), oracle.rmsnorm(x, w, 0.0), atol=1e-12)


def test_rmsnorm_bwd_matches_autograd():
    x, w, dy = r64((3, 7, 16), 3).requires_grad_(), r64((16,), 4).requires_grad_(), r64((3, 7, 16), 5)
    oracle.rmsnorm(x, w).backward(dy)
    dx, dw = oracle.rmsnorm_bwd(x.detach(), w.detach(), dy)
    assert torch.allclose(dx, x.grad, atol=1e-12) and torch.allclose(dw, w.grad, atol=1e-12)


def test_rmsnorm_equals_installed_hf():
    ml = pytest.importorskip("transformers.models.llama.modeling_llama")
    n = ml.LlamaRMSNorm(64, eps=1e-6)
    with torch.no_grad():
        n.weight.copy_(randn((64,), 6))
    x = randn((2, 9, 64), 7, dtype=torch.bfloat16)
    assert torch.equal(n.to(torch.bfloat16)(x), oracle.rmsnorm(x, n.weight.to(torch.bfloat16)))


# ------------------------------------------------------------------ RoPE
def test_rope_invariants():
    B, L, H, D = 1, 37, 3, 16
    q, k = r64((B, L, H, D), 10), r64((B, L, H, D), 11)
    pos = torch.arange(L)[None]
    cos, sin = oracle.rope_cos_sin(pos, D, 10000.0, D64)
    qr, kr = oracle.apply_rope(q, cos, sin), oracle.apply_rope(k, cos, sin)
    assert torch.allclose(qr[:, 0], q[:, 0], atol=1e-12)                       # position 0 is the identity
    pair = lambda t: t[..., :D // 2] ** 2 + t[..., D // 2:] ** 2
    assert torch.allclose(pair(qr), pair(q), atol=1e-9)                        # each (j, j + D/2) pair is rotated
    # <rope(q, m), rope(k, n)> depends on m - n only
    qq, kk = q[:, :1].expand(B, L, H, D), k[:, :1].expand(B, L, H, D)
    a, b = oracle.apply_rope(qq, cos, sin), oracle.apply_rope(kk, cos, sin)
    d1 = (a[:, 5] * b[:, 2]).sum(-1)
    d2 = (a[:, 30] * b[:, 27]).sum(-1)
    assert torch.allclose(d1, d2, atol=1e-9)
    # explicit frequency: pair j rotates by pos * base^(-2j/D)
    j, p = 3, 11
    th = p * 10000.0 ** (-2 * j / D)
    x1, x2 = q[0, p, 0, j], q[0, p, 0, j + D // 2]
    assert math.isclose(qr[0, p, 0, j].item(), (x1 * math.cos(th) - x2 * math.sin(th)).item(), rel_tol=1e-9)
    assert math.isclose(qr[0, p, 0, j + D // 2].item(), (x2 * math.cos(th) + x1 * math.sin(th)).item(), rel_tol=1e-9)


def test_rope_bwd_is_transpose_and_autograd():
    B, L, H, D = 1, 9, 2, 8
    x, dy = r64((B, L, H, D), 12).requires_grad_(), r64((B, L, H, D), 13)
    cos, sin = oracle.rope_cos_sin(torch.arange(L)[None] * 3 + 1, D, 500.0, D64)
    oracle.apply_rope(x, cos, sin).backward(dy)
    assert torch.allclose(oracle.apply_rope_bwd(dy, cos, sin), x.grad, atol=1e-12)


def test_rope_equals_installed_hf():
    ml = pytest.importorskip("transformers.models.llama.modeling_llama")
    B, L, H, D = 1, 33, 4, 32
    q, k = randn((B, H, L, D), 14), randn((B, H, L, D), 15)       # HF layout (B, H, L, D)
    pos = torch.arange(L)[None]
    cos, sin = oracle.rope_cos_sin(pos, D, 10000.0, torch.float32)
    hq, hk = ml.apply_rotary_pos_emb(q, k, cos, sin)
    assert torch.allclose(hq.transpose(1, 2), oracle.apply_rope(q.transpose(1, 2), cos, sin), atol=1e-6)
    assert torch.allclose(hk.transpose(1, 2), oracle.apply_rope(k.transpose(1, 2), cos, sin), atol=1e-6)
    cfg = ml.LlamaConfig(hidden_size=H * D, num_attention_heads=H, head_dim=D, max_position_embeddings=64)
    hcos, hsin = ml.LlamaRotaryEmbedding(cfg)(q, pos)
    assert torch.allclose(hcos, cos, atol=1e-6) and torch.allclose(hsin, sin, atol=1e-6)


# ------------------------------------------------------------------ attention
@pytest.mark.parametrize("Hq,Hkv,Lq,Lk,causal", [(4, 4, 33, 33, True), (4, 2, 40, 40, True), (4, 1, 17, 29, False),
                                                 (2, 1, 16, 24, True)])
def test_attention_fwd_vs_sdpa_and_logsumexp(Hq, Hkv, Lq, Lk, causal):
    D = 16
    q, k, v = r64((2, Lq, Hq, D), 20), r64((2, Lk, Hkv, D), 21), r64((2, Lk, Hkv, D), 22)
    o, lse = oracle.attention_fwd(q, k, v, causal=causal, block=7)
    mask = None
    if causal:
        mask = (torch.arange(Lk)[None, :] <= torch.arange(Lq)[:, None] + (Lk - Lq))
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), attn_mask=mask,
                                         enable_gqa=True).transpose(1, 2)
    assert torch.allclose(o, ref, atol=1e-10)
    kk = k.repeat_interleave(Hq // Hkv, dim=2)
    s = torch.einsum("blhd,bmhd->bhlm", q, kk) / math.sqrt(D)
    if causal:
        s = s.masked_fill(~mask, float("-inf"))
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-10)


def test_attention_is_causal_flag_of_sdpa_and_row0():
    q, k, v = r64((1, 21, 2, 8), 23), r64((1, 21, 2, 8), 24), r64((1, 21, 2, 8), 25)
    o, lse = oracle.attention_fwd(q, k, v, causal=True)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True)
    assert torch.allclose(o, ref.transpose(1, 2), atol=1e-10)
    assert torch.allclose(o[:, 0], v[:, 0], atol=1e-12)
    assert torch.allclose(lse[:, :, 0], (q[:, 0] * k[:, 0]).sum(-1) / math.sqrt(8), atol=1e-12)


@pytest.mark.parametrize("Hq,Hkv,Lq,Lk,causal", [(4, 4, 19, 19, True), (4, 2, 23, 23, True), (4, 1, 9, 14, False),
                                                 (2, 1, 12, 20, True)])
def test_attention_bwd_vs_autograd(Hq, Hkv, Lq, Lk, causal):
    D = 8
    q, k, v = (t.requires_grad_() for t in (r64((1, Lq, Hq, D), 30), r64((1, Lk, Hkv, D), 31), r64((1, Lk, Hkv, D), 32)))
    do = r64((1, Lq, Hq, D), 33)
    o, lse = oracle.attention_naive(q, k, v, causal=causal)
    o.backward(do)
    dq, dk, dv = oracle.attention_bwd(q.detach(), k.detach(), v.detach(), o.detach(), lse.detach(), do, causal=causal,
                                      block=5)
    assert torch.allclose(dq, q.grad, atol=1e-10)
    assert torch.allclose(dk, k.grad, atol=1e-10)
    assert torch.allclose(dv, v.grad, atol=1e-10)


@pytest.mark.parametrize("Hq,Hkv,Lq,Lk,causal", [(4, 4, 19, 19, True), (4, 2, 23, 23, True), (4, 1, 9, 14, False),
                                                 (2, 1, 12, 20, True)])
def test_attention_with_dropout_vs_autograd(Hq, Hkv, Lq, Lk, causal):
    """Given the mask, the dropout arithmetic is what autograd makes of softmax -> F.dropout's rule (zero or
    1 / (1 - p)) -> P V; the mask is the same however the index ranges are cut into blocks."""
    D, pdrop, seed = 8, 0.3, 0x1234ABCD5678
    q, k, v = (t.requires_grad_() for t in (r64((2, Lq, Hq, D), 30), r64((2, Lk, Hkv, D), 31), r64((2, Lk, Hkv, D), 32)))
    do = r64((2, Lq, Hq, D), 33)
    keep = oracle.dropout_keep_mask(seed, pdrop, 2, Hq, torch.arange(Lq), torch.arange(Lk))
    # the rule of torch's own dropout on the same mask
    ones = torch.ones(2, Hq, Lq, Lk, dtype=torch.float64)
    assert torch.equal(torch.where(keep, ones / (1 - pdrop), 0 * ones), keep * F.dropout(ones, pdrop, training=False) / (1 - pdrop))
    o, lse = oracle.attention_naive(q, k, v, causal=causal, keep=keep, dropout_p=pdrop)
    o.backward(do)
    o2, lse2 = oracle.attention_fwd(q.detach(), k.detach(), v.detach(), causal=causal, block=5, dropout_p=pdrop, seed=seed)
    assert torch.allclose(o2, o.detach(), atol=1e-10) and torch.allclose(lse2, lse.detach(), atol=1e-10)
    lse_plain = oracle.attention_fwd(q.detach(), k.detach(), v.detach(), causal=causal)[1]
    assert torch.allclose(lse2, lse_plain, atol=1e-12)             # lse is that of the full P
    dq, dk, dv = oracle.attention_bwd(q.detach(), k.detach(), v.detach(), o2, lse2, do, causal=causal, block=7,
                                      dropout_p=pdrop, seed=seed)
    assert torch.allclose(dq, q.grad, atol=1e-10)
    assert torch.allclose(dk, k.grad, atol=1e-10)
    assert torch.allclose(dv, v.grad, atol=1e-10)


def test_dropout_mask_properties():
    """Kept fraction 1 - p within sampling error, for every (batch, head), row and column alike; different seeds,
    heads and batches give different masks; a mask does not depend on how its index ranges are sliced."""
    L = 640
    for pdrop in (0.05, 0.1, 0.5):
        m = oracle.dropout_keep_mask(99, pdrop, 2, 3, torch.arange(L), torch.arange(L)).double()
        se = math.sqrt(pdrop * (1 - pdrop) / (L * L))
        assert (m.mean((-1, -2)) - (1 - pdrop)).abs().max() < 5 * se
        row_se = math.sqrt(pdrop * (1 - pdrop) / L)
        assert (m.mean(-1) - (1 - pdrop)).abs().max() < 6 * row_se and (m.mean(-2) - (1 - pdrop)).abs().max() < 6 * row_se
        # neighbouring entries are uncorrelated (along keys, along queries, across heads)
        c = m - (1 - pdrop)
        for a, b in ((c[..., :-1], c[..., 1:]), (c[..., :-1, :], c[..., 1:, :]), (c[:, 0], c[:, 1]), (c[0], c[1])):
            assert abs((a * b).mean().item()) < 6 * pdrop * (1 - pdrop) / math.sqrt(a.numel())
    m = oracle.dropout_keep_mask(99, 0.1, 2, 3, torch.arange(L), torch.arange(L))
    assert not torch.equal(m, oracle.dropout_keep_mask(100, 0.1, 2, 3, torch.arange(L), torch.arange(L)))
    part = oracle.dropout_keep_mask(99, 0.1, 2, 3, torch.arange(17, 300), torch.arange(401, 640))
    assert torch.equal(part, m[:, :, 17:300, 401:640])
    assert not torch.equal(m, oracle.dropout_keep_mask(99 + (1 << 32), 0.1, 2, 3, torch.arange(L), torch.arange(L)))   # all 64 seed bits count


def test_gqa_equals_mha_on_repeated_kv():
    q, k, v, do = r64((1, 15, 4, 8), 34), r64((1, 15, 2, 8), 35), r64((1, 15, 2, 8), 36), r64((1, 15, 4, 8), 37)
    o, lse = oracle.attention_fwd(q, k, v)
    kr, vr = k.repeat_interleave(2, 2), v.repeat_interleave(2, 2)
    o2, lse2 = oracle.attention_fwd(q, kr, vr)
    assert torch.allclose(o, o2, atol=1e-12) and torch.allclose(lse, lse2, atol=1e-12)
    dq, dk, dv = oracle.attention_bwd(q, k, v, o, lse, do)
    dq2, dk2, dv2 = oracle.attention_bwd(q, kr, vr, o2, lse2, do)
    assert torch.allclose(dq, dq2, atol=1e-12)
    assert torch.allclose(dk, dk2.view(1, 15, 2, 2, 8).sum(3), atol=1e-12)
    assert torch.allclose(dv, dv2.view(1, 15, 2, 2, 8).sum(3), atol=1e-12)


def test_empty_rows_when_queries_outnumber_keys():
    # causal with Lk < Lq: the first Lq - Lk queries see nothing
    q, k, v = r64((1, 10, 1, 4), 38), r64((1, 6, 1, 4), 39), r64((1, 6, 1, 4), 40)
    o, lse = oracle.attention_fwd(q, k, v, causal=True)
    assert torch.isinf(lse[0, 0, :4]).all() and (o[0, :4] == 0).all()
    assert torch.isfinite(lse[0, 0, 4:]).all()
    dq, dk, dv = oracle.attention_bwd(q, k, v, o, lse, torch.ones_like(o), causal=True)
    assert (dq[0, :4] == 0).all() and torch.isfinite(dk).all()


# ------------------------------------------------------------------ ring step
def test_ring_merge_equals_unsplit_attention_fwd_and_bwd():
    B, Lq, H, Hkv, D, NB = 1, 12, 4, 2, 8, 4
    q = r64((B, Lq, H, D), 41).requires_grad_()
    ks = [r64((B, Lq, Hkv, D), 50 + b).requires_grad_() for b in range(NB)]
    vs = [r64((B, Lq, Hkv, D), 60 + b).requires_grad_() for b in range(NB)]
    do = r64((B, Lq, H, D), 42)
    k_all, v_all = torch.cat(ks[1:] + ks[:1], 1), torch.cat(vs[1:] + vs[:1], 1)   # diagonal block last
    o_ref, lse_ref = oracle.attention_naive(q, k_all, v_all, causal=True)
    o_ref.backward(do)
    det = lambda ts: [t.detach() for t in ts]
    o, lse = oracle.ring_attention_fwd(q.detach(), det(ks), det(vs), causal_block=0)
    assert torch.allclose(o, o_ref, atol=1e-10) and torch.allclose(lse, lse_ref, atol=1e-10)
    dq, dks, dvs = oracle.ring_attention_bwd(q.detach(), det(ks), det(vs), o, lse, do, causal_block=0)
    assert torch.allclose(dq, q.grad, atol=1e-10)
    for b in range(NB):
        assert torch.allclose(dks[b], ks[b].grad, atol=1e-10) and torch.allclose(dvs[b], vs[b].grad, atol=1e-10)


def test_lse_merge_algebra():
    o1, l1, o2, l2, o3, l3 = (r64((1, 5, 2, 4), 70), r64((1, 2, 5), 71), r64((1, 5, 2, 4), 72), r64((1, 2, 5), 73),
                              r64((1, 5, 2, 4), 74), r64((1, 2, 5), 75))
    a, la = oracle.lse_merge(*oracle.lse_merge(o1, l1, o2, l2), o3, l3)
    b, lb = oracle.lse_merge(o1, l1, *oracle.lse_merge(o2, l2, o3, l3))
    c, lc = oracle.lse_merge(*oracle.lse_merge(o3, l3, o1, l1), o2, l2)
    assert torch.allclose(a, b, atol=1e-12) and torch.allclose(a, c, atol=1e-12)      # associative, commutative
    assert torch.allclose(la, lb, atol=1e-12) and torch.allclose(la, lc, atol=1e-12)
    ninf = torch.full_like(l2, float("-inf"))
    d, ld = oracle.lse_merge(o1, l1, o2, ninf)                                          # -inf side is the identity
    assert torch.equal(d, o1) and torch.equal(ld, l1)
    # the alternative form quoted for the update: o - sigmoid(lb - l) * (o - ob)
    e, le = oracle.lse_merge(o1, l1, o2, l2)
    sg = torch.sigmoid(l2 - l1).permute(0, 2, 1)[..., None]
    assert torch.allclose(e, o1 - sg * (o1 - o2), atol=1e-12)
    assert torch.allclose(le, l1 + torch.log1p(torch.exp(l2 - l1)), atol=1e-12)


# ------------------------------------------------------------------ linears, SwiGLU, layer
def test_linear_vs_functional_and_autograd():
    x, w, b = r64((1, 11, 6), 80).requires_grad_(), r64((9, 6), 81).requires_grad_(), r64((9,), 82).requires_grad_()
    dy = r64((1, 11, 9), 83)
    y = oracle.linear_fwd(x, w, b)
    assert torch.allclose(y, F.linear(x, w, b), atol=1e-12)
    y.backward(dy)
    dx, dw, db = oracle.linear_bwd(x.detach(), w.detach(), dy, has_bias=True)
    assert torch.allclose(dx, x.grad, atol=1e-12) and torch.allclose(dw, w.grad, atol=1e-12)
    assert torch.allclose(db, b.grad, atol=1e-12)


def test_swiglu_mlp_equals_installed_hf_llama_mlp():
    ml = pytest.importorskip("transformers.models.llama.modeling_llama")
    cfg = ml.LlamaConfig(hidden_size=16, intermediate_size=24, num_attention_heads=2)
    mlp = ml.LlamaMLP(cfg).to(D64)
    x = r64((1, 7, 16), 84)
    w_gu = torch.cat((mlp.gate_proj.weight, mlp.up_proj.weight), 0).detach()       # gate = rows [0, i), up = rows [i, 2i)
    assert torch.allclose(oracle.swiglu_mlp_fwd(x, w_gu, mlp.down_proj.weight.detach()), mlp(x), atol=1e-12)


def test_swiglu_and_mlp_bwd_vs_autograd():
    x, wgu, wd = (t.requires_grad_() for t in (r64((1, 5, 8), 85), r64((12, 8), 86), r64((8, 6), 87)))
    dy = r64((1, 5, 8), 88)
    oracle.swiglu_mlp_fwd(x, wgu, wd).backward(dy)
    dx, dwgu, dwd = oracle.swiglu_mlp_bwd(x.detach(), wgu.detach(), wd.detach(), dy)
    assert torch.allclose(dx, x.grad, atol=1e-12) and torch.allclose(dwgu, wgu.grad, atol=1e-12)
    assert torch.allclose(dwd, wd.grad, atol=1e-12)


def test_packed_qkv_equals_three_linears():
    H, Hkv, D, d = 4, 2, 8, 16
    x, w = r64((1, 6, d), 89), r64(((H + 2 * Hkv) * D, d), 90)
    q, k, v = oracle.split_qkv(oracle.linear_fwd(x, w), H, Hkv, D)
    assert torch.allclose(q.reshape(1, 6, -1), F.linear(x, w[:H * D]), atol=1e-12)
    assert torch.allclose(k.reshape(1, 6, -1), F.linear(x, w[H * D:(H + Hkv) * D]), atol=1e-12)
    assert torch.allclose(v.reshape(1, 6, -1), F.linear(x, w[(H + Hkv) * D:]), atol=1e-12)


def test_decoder_layer_explicit_bwd_vs_autograd_and_hf_layer():
    H, Hkv, D, d, i, L = 4, 2, 8, 32, 40, 13
    p = {"ln1": 1 + r64((d,), 91, 0.1), "w_qkv": r64(((H + 2 * Hkv) * D, d), 92, 0.2), "w_o": r64((d, H * D), 93, 0.2),
         "ln2": 1 + r64((d,), 94, 0.1), "w_gate_up": r64((2 * i, d), 95, 0.2), "w_down": r64((d, i), 96, 0.2)}
    x, dy = r64((1, L, d), 97), r64((1, L, d), 98)
    leaves = {k: v.clone().requires_grad_() for k, v in p.items()}
    xl = x.clone().requires_grad_()
    y = oracle.decoder_layer_fwd(xl, leaves, H, Hkv, D, differentiable=True)
    y.backward(dy)
    y2, g = oracle.decoder_layer_fwd_bwd(x, p, dy, H, Hkv, D)
    assert torch.allclose(y, y2, atol=1e-10)
    assert torch.allclose(g["x"], xl.grad, atol=1e-9)
    for k in p:
        assert torch.allclose(g[k], leaves[k].grad, atol=1e-9), k
    # the same weights in the installed transformers' LlamaDecoderLayer (eager attention)
    ml = pytest.importorskip("transformers.models.llama.modeling_llama")
    cfg = ml.LlamaConfig(hidden_size=d, intermediate_size=i, num_attention_heads=H, num_key_value_heads=Hkv, head_dim=D,
                         rms_norm_eps=1e-6, attention_bias=False, mlp_bias=False)
    cfg._attn_implementation = "eager"
    layer = ml.LlamaDecoderLayer(cfg, 0).to(D64)
    with torch.no_grad():
        layer.input_layernorm.weight.copy_(p["ln1"])
        layer.post_attention_layernorm.weight.copy_(p["ln2"])
        layer.self_attn.q_proj.weight.copy_(p["w_qkv"][:H * D])
        layer.self_attn.k_proj.weight.copy_(p["w_qkv"][H * D:(H + Hkv) * D])
        layer.self_attn.v_proj.weight.copy_(p["w_qkv"][(H + Hkv) * D:])
        layer.self_attn.o_proj.weight.copy_(p["w_o"])
        layer.mlp.gate_proj.weight.copy_(p["w_gate_up"][:i])
        layer.mlp.up_proj.weight.copy_(p["w_gate_up"][i:])
        layer.mlp.down_proj.weight.copy_(p["w_down"])
    pos = torch.arange(L)[None]
    cos, sin = oracle.rope_cos_sin(pos, D, 10000.0, D64)
    mask = torch.full((L, L), float("-inf"), dtype=D64).triu(1)[None, None]
    out = layer(x, attention_mask=mask, position_ids=pos, position_embeddings=(cos, sin))
    out = out[0] if isinstance(out, tuple) else out
    assert torch.allclose(out, y2, atol=1e-5)      # HF's eager softmax runs in fp32


# ------------------------------------------------------------------ the sampled checker used at full sizes
@pytest.mark.parametrize("Hq,Hkv,Lq,Lk", [(4, 2, 300, 300), (2, 1, 130, 390)])
def test_sampled_checker_accepts_the_oracle_and_rejects_mistakes(Hq, Hkv, Lq, Lk):
    from sampled import edge_samples, sampled_checks
    D = 32
    q, do = randn((1, Lq, Hq, D), 90), randn((1, Lq, Hq, D), 91)
    k, v = randn((1, Lk, Hkv, D), 92), randn((1, Lk, Hkv, D), 93)
    o, lse = oracle.attention_fwd(q, k, v, causal=True)
    dq, dk, dv = oracle.attention_bwd(q, k, v, o, lse, do, causal=True)
    rows, cols = edge_samples(Lq, 5, 1), edge_samples(Lk, 5, 2)
    args = [q[0], k[0], v[0], do[0], o[0], lse[0], dq[0], dk[0], dv[0]]
    sampled_checks(*args, True, rows, cols)
    for idx, bad in ((4, -o[0]), (6, dq[0] * 1.1), (7, dk[0].flip(0)), (8, dv[0] + 0.05 * dv[0].abs().max())):
        wrong = list(args)
        wrong[idx] = bad
        with pytest.raises(AssertionError):
            sampled_checks(*wrong, True, rows, cols)


def test_cross_entropy_equals_torch_and_its_autograd():
    g = torch.Generator().manual_seed(5)
    T, V = 37, 101
    x = torch.randn(T, V, generator=g, dtype=torch.float64) * 3
    y = torch.randint(0, V, (T,), generator=g)
    y[::5] = -100
    loss, losses, lse, dx = oracle.cross_entropy_fwd_bwd(x, y, grad_loss=0.7)
    xr = x.clone().requires_grad_(True)
    ref = torch.nn.functional.cross_entropy(xr, y, ignore_index=-100)
    (ref * 0.7).backward()
    assert torch.allclose(loss, ref.detach(), rtol=1e-12)
    assert torch.allclose(dx, xr.grad, rtol=1e-10, atol=1e-14)
    assert torch.allclose(losses, torch.nn.functional.cross_entropy(x, y, ignore_index=-100, reduction="none"), rtol=1e-12)
    assert torch.allclose(lse, torch.logsumexp(x, -1))
    assert dx.sum(-1).abs().max() < 1e-12 and (dx[::5] == 0).all()


def test_adamw_step_is_torch_adamw():
    """Parameter and both moments over several steps against torch.optim.AdamW in fp64; zero gradient: decay only."""
    g = torch.Generator().manual_seed(321)
    p0 = torch.randn(257, generator=g, dtype=torch.float64)
    grads = [torch.randn(257, generator=g, dtype=torch.float64) for _ in range(5)]
    hp = dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    ref = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([ref], **hp)
    p, m, v = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    for step, gr in enumerate(grads, 1):
        ref.grad = gr.clone()
        opt.step()
        p, m, v = oracle.adamw_step(p, gr, m, v, step, **hp)
        assert torch.allclose(p, ref.detach(), rtol=1e-12, atol=1e-14)
        assert torch.allclose(m, opt.state[ref]["exp_avg"], rtol=1e-12, atol=1e-14)
        assert torch.allclose(v, opt.state[ref]["exp_avg_sq"], rtol=1e-12, atol=1e-14)
    z = torch.zeros_like(p0)
    p1, m1, v1 = oracle.adamw_step(p0, z, z, z, 1, lr=1e-2, weight_decay=0.5)
    assert torch.allclose(p1, p0 * (1 - 1e-2 * 0.5)) and not m1.any() and not v1.any()
