"""GPU parity: RMSNorm, RoPE, SwiGLU and the LSE merge vs. the CPU oracle."""
import pytest
import torch

from conftest import TOL_BF16, TOL_F32, TOL_LSE, assert_parity, randn, rel_err
import odysseus_oracle as oracle

pytestmark = pytest.mark.gpu
DTYPES = pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])


def _tol(dtype):
    return TOL_BF16 if dtype == torch.bfloat16 else TOL_F32


@DTYPES
@pytest.mark.parametrize("T,d", [(7, 512), (2048, 512), (513, 4096), (3, 8192), (5, 16384)])
def test_rmsnorm(T, d, dtype, dev):
    from odysseus_transformer_amd import ops
    x = randn((1, T, d), 1, dtype=dtype)
    w = (1.0 + randn((d,), 2, std=0.02)).to(dtype)
    dy = randn((1, T, d), 3, dtype=dtype)
    y_ref = oracle.rmsnorm(x.float(), w.float())
    y, rstd = ops.rmsnorm_fwd(x.to(dev), w.to(dev), 1e-6)
    assert rel_err(y, y_ref) <= _tol(dtype)
    n = 256 * (8 if dtype == torch.bfloat16 else 4) * 4
    if d <= n:
        dx_ref, dw_ref = oracle.rmsnorm_bwd(x.float(), w.float(), dy.float())
        dx, dw = ops.rmsnorm_bwd(x.to(dev), w.to(dev), rstd, dy.to(dev))
        assert rel_err(dx, dx_ref) <= _tol(dtype)
        assert rel_err(dw, dw_ref) <= _tol(dtype)
        # with the gradient of the residual path added inside the kernel
        skip = randn((1, T, d), 4, dtype=dtype)
        dx2, dw2 = ops.rmsnorm_bwd(x.to(dev), w.to(dev), rstd, dy.to(dev), dx_add=skip.to(dev))
        assert rel_err(dx2, dx_ref.float() + skip.float()) <= _tol(dtype)
        assert torch.equal(dw2, dw)
    else:
        # rows longer than the backward kernel holds in registers are refused, not mangled
        from odysseus_transformer_amd._lib import OdysseusHipError
        with pytest.raises(OdysseusHipError) as e:
            ops.rmsnorm_bwd(x.to(dev), w.to(dev), rstd, dy.to(dev))
        assert e.value.code == -2


@DTYPES
@pytest.mark.parametrize("B,L,H,Hkv,D", [(1, 2048, 8, 8, 64), (2, 300, 4, 1, 128), (1, 4096, 4, 4, 128)])
def test_rope(B, L, H, Hkv, D, dtype, dev):
    from odysseus_transformer_amd import ops
    qkv = randn((B, L, H + 2 * Hkv, D), 9, dtype=dtype)
    pos = torch.arange(L)[None].expand(B, L)
    cos, sin = oracle.rope_cos_sin(pos, D, 10000.0, torch.float32)
    ref = qkv.float().clone()
    ref[:, :, :H + Hkv] = oracle.apply_rope(ref[:, :, :H + Hkv], cos, sin)
    g = qkv.to(dev).clone()
    ops.rope_(g, H + Hkv, None, 10000.0)
    assert rel_err(g, ref) <= _tol(dtype)
    assert torch.equal(g[:, :, H + Hkv:].cpu(), qkv[:, :, H + Hkv:])          # v untouched
    # explicit position ids == implicit arange; inverse undoes the rotation
    g2 = qkv.to(dev).clone()
    ops.rope_(g2, H + Hkv, pos.to(dev), 10000.0)
    assert torch.equal(g2, g)
    ops.rope_(g2, H + Hkv, pos.to(dev), 10000.0, inverse=True)
    assert rel_err(g2, qkv.float()) <= _tol(dtype)
    # backward == oracle's explicit backward
    dref = qkv.float().clone()
    dref[:, :, :H + Hkv] = oracle.apply_rope_bwd(dref[:, :, :H + Hkv], cos, sin)
    g3 = qkv.to(dev).clone()
    ops.rope_(g3, H + Hkv, None, 10000.0, inverse=True)
    assert rel_err(g3, dref) <= _tol(dtype)


def test_rope_far_positions_fp32(dev):
    """Position ids far from zero: the angle is formed in fp32 exactly as on the host."""
    from odysseus_transformer_amd import ops
    B, L, H, D = 1, 64, 2, 128
    x = randn((B, L, H, D), 4)
    pos = (torch.arange(L) * 2053 + 100000)[None]
    cos, sin = oracle.rope_cos_sin(pos, D, 10000.0, torch.float32)
    ref = oracle.apply_rope(x, cos, sin)
    g = x.to(dev).clone()
    ops.rope_(g, H, pos.to(dev), 10000.0)
    assert rel_err(g, ref) <= TOL_F32


@DTYPES
@pytest.mark.parametrize("T,I", [(5, 1376), (2048, 1376), (300, 11008)])
def test_swiglu(T, I, dtype, dev):
    from odysseus_transformer_amd import ops
    gu = randn((1, T, 2 * I), 21, dtype=dtype)
    dh = randn((1, T, I), 22, dtype=dtype)
    h_ref = oracle.swiglu(gu.float())
    dgu_ref = oracle.swiglu_bwd(gu.float(), dh.float())
    h = ops.swiglu_fwd(gu.to(dev))
    dgu = ops.swiglu_bwd(gu.to(dev), dh.to(dev))
    assert rel_err(h, h_ref) <= _tol(dtype)
    assert rel_err(dgu, dgu_ref) <= _tol(dtype)


@DTYPES
def test_lse_merge(dtype, dev):
    from odysseus_transformer_amd import ops
    B, L, H, D = 2, 130, 4, 128
    out = randn((B, L, H, D), 31)
    lse = randn((B, H, L), 32, std=3.0)
    ob = randn((B, L, H, D), 33, dtype=dtype)
    lb = randn((B, H, L), 34, std=3.0)
    lse[0, 0, :5] = float("-inf")          # running side empty
    lb[0, 1, :5] = float("-inf")           # block side empty
    lse[1, 2, 7] = lb[1, 2, 7] = float("-inf")   # both empty
    o_ref, l_ref = oracle.lse_merge(out, lse, ob.float(), lb)
    og, lg = out.to(dev).clone(), lse.to(dev).clone()
    ops.lse_merge_(og, lg, ob.to(dev), lb.to(dev))
    assert rel_err(og, o_ref) <= 1e-5
    assert torch.allclose(lg.cpu(), l_ref, atol=1e-5, rtol=1e-5)
    assert torch.isinf(lg[1, 2, 7]) and (og[1, 7, 2] == 0).all()


def test_ring_step_equals_unsplit_attention(dev):
    """Block attention + merge over a partition of the keys == attention over all keys,
    forward and every gradient (the invariant that pins the ring step)."""
    from odysseus_transformer_amd import ops
    B, Lq, H, Hkv, D, NB = 1, 256, 4, 2, 128, 3
    dt = torch.bfloat16
    q = randn((B, Lq, H, D), 41, dtype=dt)
    ks = [randn((B, Lq, Hkv, D), 50 + b, dtype=dt) for b in range(NB)]
    vs = [randn((B, Lq, Hkv, D), 60 + b, dtype=dt) for b in range(NB)]
    do = randn((B, Lq, H, D), 42, dtype=dt)
    # oracle: the causal diagonal block is block 0; the others are fully visible.  As one
    # attention call that is keys = [blocks 1.., block 0] with the bottom-right causal mask.
    k_all = torch.cat(ks[1:] + ks[:1], 1).float()
    v_all = torch.cat(vs[1:] + vs[:1], 1).float()
    o_ref, lse_ref = oracle.attention_fwd(q.float(), k_all, v_all, causal=True)
    dq_ref, dk_ref, dv_ref = oracle.attention_bwd(q.float(), k_all, v_all, o_ref, lse_ref, do.float(), causal=True)
    o2, l2 = oracle.ring_attention_fwd(q.float(), [k.float() for k in ks], [v.float() for v in vs], causal_block=0)
    assert rel_err(o2, o_ref) <= 1e-5 and torch.allclose(l2, lse_ref, atol=1e-5)
    # device ring step
    qg, dog = q.to(dev), do.to(dev)
    out = torch.zeros((B, Lq, H, D), dtype=torch.float32, device=dev)
    lse = torch.full((B, H, Lq), float("-inf"), dtype=torch.float32, device=dev)
    for b in range(NB):
        ob, lb = ops.attn_fwd(qg, ks[b].to(dev), vs[b].to(dev), causal=(b == 0))
        ops.lse_merge_(out, lse, ob, lb)
    assert_parity(out, o_ref, TOL_BF16, "out")
    assert torch.allclose(lse.cpu(), lse_ref, atol=TOL_LSE, rtol=TOL_LSE)
    out_bf = out.to(dt)
    dq = torch.zeros_like(qg)
    dks, dvs = [], []
    for b in range(NB):
        _, dk, dv = ops.attn_bwd(qg, ks[b].to(dev), vs[b].to(dev), out_bf, lse, dog, causal=(b == 0), dq=dq,
                                 accumulate_dq=(b > 0))
        dks.append(dk)
        dvs.append(dv)
    assert_parity(dq, dq_ref, TOL_BF16, "dq")
    assert_parity(torch.cat(dks[1:] + dks[:1], 1), dk_ref, TOL_BF16, "dk")
    assert_parity(torch.cat(dvs[1:] + dvs[:1], 1), dv_ref, TOL_BF16, "dv")


def test_ring_backward_fp32_dq_and_reused_query_side(dev):
    """Over many key blocks the bf16 running dq is rounded after every block; the fp32 one is exact and is
    rounded once.  Reusing the query-side scratch of the first block's call changes nothing."""
    from odysseus_transformer_amd import ops
    B, Lq, H, D, NB = 1, 320, 2, 128, 6
    dt = torch.bfloat16
    q, do = randn((B, Lq, H, D), 70, dtype=dt), randn((B, Lq, H, D), 71, dtype=dt)
    ks = [randn((B, 192, H, D), 72 + b, dtype=dt) for b in range(NB)]
    vs = [randn((B, 192, H, D), 82 + b, dtype=dt) for b in range(NB)]
    o_ref, l_ref = oracle.ring_attention_fwd(q.float(), [k.float() for k in ks], [v.float() for v in vs], causal_block=None)
    dq_ref, dk_ref, dv_ref = oracle.ring_attention_bwd(q.float(), [k.float() for k in ks], [v.float() for v in vs], o_ref,
                                                       l_ref, do.float(), causal_block=None)
    qg, dog = q.to(dev), do.to(dev)
    kg, vg = [k.to(dev) for k in ks], [v.to(dev) for v in vs]
    out, lse = o_ref.to(dt).to(dev), l_ref.to(dev)
    runs = {}
    for name, f32, reuse in (("bf16", False, False), ("fp32", True, False), ("fp32_reuse", True, True)):
        dq = torch.empty(qg.shape, dtype=torch.float32 if f32 else dt, device=dev)
        ws = ops.attn_bwd_workspace(qg, kg[0])
        dks = []
        for b in range(NB):
            _, dk, _ = ops.attn_bwd(qg, kg[b], vg[b], out, lse, dog, causal=False, dq=dq, accumulate_dq=(b > 0),
                                    workspace=ws, reuse_query_side=(reuse and b > 0))
            dks.append(dk)
        runs[name] = (dq.float().cpu(), dks)
    assert torch.equal(runs["fp32"][0], runs["fp32_reuse"][0])
    assert all(torch.equal(a, b) for a, b in zip(runs["fp32"][1], runs["fp32_reuse"][1]))
    e_bf16, e_f32 = rel_err(runs["bf16"][0], dq_ref), rel_err(runs["fp32"][0], dq_ref)
    assert e_f32 <= TOL_BF16 / 4 and e_f32 < e_bf16, (e_f32, e_bf16)
    for b in range(NB):
        assert_parity(runs["fp32"][1][b], dk_ref[b], TOL_BF16, f"dk block {b}")
    with pytest.raises(ValueError):
        ops.attn_bwd(qg, kg[0], vg[0], out, lse, dog, causal=False, reuse_query_side=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_ring_blocks_autograd_function(dtype, dev):
    """ops.ring_blocks_attn (forward merge + backward over blocks under autograd) vs. the oracle's ring loop."""
    from odysseus_transformer_amd import ops
    B, Lq, H, Hkv, D, NB = 1, 200, 4, 2, 64, 3
    tol = TOL_BF16 if dtype == torch.bfloat16 else 1e-4
    q = randn((B, Lq, H, D), 71, dtype=dtype)
    ks = [randn((B, Lq, Hkv, D), 72 + b, dtype=dtype) for b in range(NB)]
    vs = [randn((B, Lq, Hkv, D), 82 + b, dtype=dtype) for b in range(NB)]
    do = randn((B, Lq, H, D), 70, dtype=dtype)
    f = lambda ts: [t.float() for t in ts]
    o_ref, l_ref = oracle.ring_attention_fwd(q.float(), f(ks), f(vs), causal_block=1)
    dq_ref, dk_ref, dv_ref = oracle.ring_attention_bwd(q.float(), f(ks), f(vs), o_ref, l_ref, do.float(), causal_block=1)
    qg = q.to(dev).requires_grad_()
    kg = [t.to(dev).requires_grad_() for t in ks]
    vg = [t.to(dev).requires_grad_() for t in vs]
    out, lse = ops.ring_blocks_attn(qg, kg, vg, causal_block=1)
    out.backward(do.to(dev))
    assert_parity(out, o_ref, tol, "out")
    assert torch.allclose(lse.cpu(), l_ref, atol=TOL_LSE, rtol=TOL_LSE)
    assert_parity(qg.grad, dq_ref, tol, "dq")
    for b in range(NB):
        assert_parity(kg[b].grad, dk_ref[b], tol, f"dk block {b}")
        assert_parity(vg[b].grad, dv_ref[b], tol, f"dv block {b}")
