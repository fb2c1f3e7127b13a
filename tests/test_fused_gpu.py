"""The linears that carry their elementwise neighbour in the epilogue (residual add, SwiGLU forward,
SwiGLU backward) against the unfused kernels (bit for bit where the arithmetic is the same) and the
oracle, on shapes that take the fused kernel and on shapes that fall back to two kernels; and the
decoder layer built from them against the one-kernel-per-step layer."""
import types

import pytest
import torch

from conftest import TOL_BF16, TOL_F32, assert_parity, randn, rel_err
import odysseus_oracle as oracle

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _kernels_of(fn):
    from odysseus_transformer_amd import _lib
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    _lib.profile_collect()
    out = fn()
    torch.cuda.synchronize()
    names = sorted(_lib.profile_collect())
    _lib.profile_enable(False)
    return out, names


@pytest.mark.parametrize("M,N,K,dtype,fused", [(4096, 4096, 512, BF, True), (8192, 4096, 328, BF, False),
                                               (300, 520, 136, BF, False), (256, 512, 64, torch.float32, False)])
def test_linear_residual(M, N, K, dtype, fused, dev):
    from odysseus_transformer_amd import ops
    print(f"linear_residual M={M} N={N} K={K} {dtype}", flush=True)
    x, w, r = randn((M, K), 1, dtype=dtype), randn((N, K), 2, std=0.05, dtype=dtype), randn((M, N), 3, dtype=dtype)
    y, names = _kernels_of(lambda: ops.linear_residual(x.to(dev), w.to(dev), r.to(dev)))
    assert ("gemm_bf16_nt_residual" in names) == fused, names
    ref = oracle.linear_fwd(x.float(), w.float()) + r.float()
    assert_parity(y, ref, 4e-3 if dtype == BF else TOL_F32, "y")       # one rounding of the sum: half a bf16 ulp


@pytest.mark.parametrize("T,I,K,fused", [(512, 1024, 512, True), (4096, 11008, 256, True), (512, 1376, 512, False),
                                         (200, 344, 136, False)])
def test_linear_swiglu_forward_and_backward(T, I, K, fused, dev):
    from odysseus_transformer_amd import ops
    print(f"linear_swiglu T={T} I={I} K={K}", flush=True)
    x, wgu = randn((T, K), 4, dtype=BF).to(dev), randn((2 * I, K), 5, std=0.05, dtype=BF).to(dev)
    (gu, h), names = _kernels_of(lambda: ops.linear_swiglu(x, wgu))
    assert ("gemm_bf16_nt_swiglu" in names) == fused, names
    assert ("swiglu_fwd" in names) != fused
    gu_ref = ops.gemm(ops.GEMM_NT, x, wgu)
    assert torch.equal(gu, gu_ref), "gate_up differs from the plain product"
    assert torch.equal(h, ops.swiglu_fwd(gu_ref)), "h differs from the stand-alone SwiGLU kernel"
    assert_parity(h, oracle.swiglu(oracle.linear_fwd(x.float().cpu(), wgu.float().cpu())), TOL_BF16, "h")
    # backward: d_gate_up from dy and the down weight (d_model = K here)
    dy, wd = randn((T, K), 6, dtype=BF).to(dev), randn((K, I), 7, std=0.05, dtype=BF).to(dev)
    fused_bwd = fused and I % 256 == 0
    dgu, names = _kernels_of(lambda: ops.linear_dgrad_swiglu(dy, wd, gu))
    assert ("gemm_bf16_nn_swiglu_bwd" in names) == fused_bwd, names
    dh = ops.gemm(ops.GEMM_NN, dy, wd)
    assert torch.equal(dgu, ops.swiglu_bwd(gu, dh)), "d_gate_up differs from the two-kernel path"
    dgu_ref = oracle.swiglu_bwd(gu.float().cpu(), oracle.linear_fwd(dy.float().cpu(), wd.float().cpu().t()))
    assert_parity(dgu, dgu_ref, TOL_BF16, "d_gate_up")


def test_fused_entry_points_validate(dev):
    from odysseus_transformer_amd import ops
    from odysseus_transformer_amd._lib import OdysseusHipError
    x = torch.zeros(256, 64, dtype=BF, device=dev)
    with pytest.raises(ValueError):
        ops.linear_residual(x, torch.zeros(128, 64, dtype=BF, device=dev), torch.zeros(256, 64, dtype=BF, device=dev))
    with pytest.raises(TypeError):
        ops.linear_swiglu(x, torch.zeros(128, 64, device=dev))
    with pytest.raises(ValueError):
        ops.linear_dgrad_swiglu(x, torch.zeros(64, 32, dtype=BF, device=dev), torch.zeros(256, 48, dtype=BF, device=dev))
    with pytest.raises(RuntimeError):
        ops.linear_swiglu(x.cpu(), torch.zeros(128, 64, dtype=BF))


def _config(d, H, Hkv, D, i):
    return types.SimpleNamespace(hidden_size=d, num_attention_heads=H, num_key_value_heads=Hkv, head_dim=D,
                                 intermediate_size=i, hidden_act="silu", attention_dropout=0.0, rms_norm_eps=1e-6,
                                 rope_theta=10000.0, max_position_embeddings=1 << 20, pretraining_tp=1,
                                 num_hidden_layers=1)


@pytest.mark.parametrize("L,d,H,Hkv,D,i,dtype", [(1024, 1024, 4, 2, 128, 2816, BF), (520, 512, 4, 1, 128, 1408, BF),
                                                 (256, 512, 8, 8, 64, 1376, torch.float32)],
                         ids=["fused_kernels", "ragged_fallbacks", "fp32"])
def test_fused_layer_matches_the_unfused_layer_and_the_oracle(L, d, H, Hkv, D, i, dtype, dev):
    from odysseus_transformer_amd.decoder.odysseus import OdysseusDecoderLayer
    tol = TOL_BF16 if dtype == BF else TOL_F32
    cfg = _config(d, H, Hkv, D, i)
    fused, plain = OdysseusDecoderLayer(cfg, fused=True).to(dtype).to(dev), OdysseusDecoderLayer(cfg, fused=False).to(dtype).to(dev)
    with torch.no_grad():
        for k, (pf, pp) in enumerate(zip(fused.parameters(), plain.parameters())):
            v = randn(tuple(pf.shape), 100 + k, std=0.02, dtype=dtype).to(dev)
            if pf.dim() == 1:
                v = v + 1.0
            pf.copy_(v)
            pp.copy_(v)
    x, dy = randn((1, L, d), 200, dtype=dtype), randn((1, L, d), 201, dtype=dtype)
    pos = torch.arange(L, device=dev)[None]
    res = []
    for layer in (fused, plain):
        xg = x.to(dev).requires_grad_(True)
        (y, names) = _kernels_of(lambda: layer(xg, position_ids=pos))
        y.backward(dy.to(dev))
        torch.cuda.synchronize()
        res.append((y.detach(), xg.grad, [p.grad for p in layer.parameters()], names))
    (yf, dxf, gf, nf), (yp, dxp, gp, npl) = res
    assert "swiglu_fwd" in npl
    if dtype == BF and L % 256 == 0:
        # (the residual epilogue needs at least 128 tiles of 256 x 256, i.e. a layer of benchmark size;
        # test_linear_residual covers it, here the add rides on the accumulating 128 x 128 kernel)
        assert "swiglu_fwd" not in nf and "swiglu_bwd" not in nf and "gemm_bf16_nt_swiglu" in nf, nf
    # the fused layer rounds each sum once where the unfused one rounds twice: close, not identical
    assert rel_err(yf, yp.float()) <= tol / 2 and rel_err(dxf, dxp.float()) <= tol / 2
    for a, b in zip(gf, gp):
        assert rel_err(a, b.float()) <= tol / 2
    p = dict(zip(("w_qkv", "w_o", "w_gate_up", "w_down", "ln1", "ln2"),
                 (fused.self_attn.qkv_proj.weight, fused.self_attn.o_proj.weight, fused.mlp.gate_up_proj.weight,
                  fused.mlp.down_proj.weight, fused.input_layernorm.weight, fused.post_attention_layernorm.weight)))
    y_ref, g_ref = oracle.decoder_layer_fwd_bwd(x.float(), {k: v.detach().float().cpu() for k, v in p.items()}, dy.float(),
                                                H, Hkv, D)
    assert_parity(yf, y_ref, tol, "y")
    assert_parity(dxf, g_ref["x"], tol, "dx")
    for k, v in p.items():
        assert rel_err(v.grad, g_ref[k]) <= tol, k


# ----------------------------------------------------------------------------------------------
# rotary embedding inside the QKV projection and the attention backward
# ----------------------------------------------------------------------------------------------
def _rope_ref(x4, pos, base=10000.0):
    """fp32 rotation of (B, L, H, D) by the oracle's cos / sin."""
    cos, sin = oracle.rope_cos_sin(pos, x4.shape[-1], base, torch.float32)
    return oracle.apply_rope(x4.float(), cos, sin)


def test_rope_table_holds_the_rounded_cos_and_sin(dev):
    from odysseus_transformer_amd import ops
    pos = torch.tensor([[0, 1, 5, 1000, 65535, 1048575]])
    t = ops.rope_table(pos.to(dev), 6, 128, 10000.0).float().cpu()
    cos, sin = oracle.rope_cos_sin(pos, 128, 10000.0, torch.float32)       # (1, 6, 128): [freqs, freqs]
    assert (t[:, 0::2] - cos[0, :, :64]).abs().max() <= 2 ** -8            # bf16 rounding of values in [-1, 1]
    assert (t[:, 1::2] - sin[0, :, :64]).abs().max() <= 2 ** -8
    t2 = ops.rope_table(None, 4, 128, 10000.0, device=dev).float().cpu()   # no positions: the row index
    cos, sin = oracle.rope_cos_sin(torch.arange(4)[None], 128, 10000.0, torch.float32)
    assert (t2[:, 0::2] - cos[0, :, :64]).abs().max() <= 2 ** -8


@pytest.mark.parametrize("M,N,K,n_rot", [(512, 768, 256, 4), (256, 1536, 4096, 8), (300, 384, 200, 2), (512, 512, 320, 0)])
def test_linear_rope_against_the_product_followed_by_the_rotation(M, N, K, n_rot, dev):
    """Fused kernel (whole 256 x 256 tiles, K a multiple of 64) and the two-kernel path for other shapes."""
    from odysseus_transformer_amd import ops
    x = randn((M, K), 9300, dtype=torch.bfloat16)
    w = randn((N, K), 9301, std=0.05, dtype=torch.bfloat16)
    pos = torch.randint(0, 40000, (1, M), generator=torch.Generator().manual_seed(9302))
    table = ops.rope_table(pos.to(dev), M, 128, 10000.0)
    y = ops.linear_rope(x.to(dev), w.to(dev), table, n_rot, 128)
    y_ref = oracle.linear_fwd(x.float(), w.float()).view(1, M, N // 128, 128)
    y_ref = torch.cat((_rope_ref(y_ref[:, :, :n_rot], pos), y_ref[:, :, n_rot:]), dim=2).reshape(M, N)
    assert_parity(y, y_ref, 1e-2, "rotated projection")     # bf16 cos / sin and one (fused) or two roundings


@pytest.mark.parametrize("L,Hq,Hkv,B", [(512, 4, 4, 1), (300, 4, 1, 1), (260, 2, 2, 2), (1024, 8, 2, 1)])
def test_attention_backward_with_the_inverse_rotation_in_its_epilogues(L, Hq, Hkv, B, dev):
    """dq and dk of ody_attn_bwd_rope against ody_attn_bwd followed by the inverse rotation: the one-kernel-per-key-head
    and the per-query-head (group sum) variants of the dK / dV kernel, ragged lengths, two batches."""
    from odysseus_transformer_amd import ops
    D = 128
    q, k, v, do = (randn((B, L, h, D), 9400 + n, dtype=torch.bfloat16).to(dev) for n, h in enumerate((Hq, Hkv, Hkv, Hq)))
    pos = torch.randint(0, 100000, (B, L), generator=torch.Generator().manual_seed(9404)).to(dev)
    out, lse = ops.attn_fwd(q, k, v, causal=True)
    dq0, dk0, dv0 = ops.attn_bwd(q, k, v, out, lse, do, causal=True)
    ops.rope_(dq0, Hq, pos, 10000.0, inverse=True)
    ops.rope_(dk0, Hkv, pos, 10000.0, inverse=True)
    table = ops.rope_table(pos, B * L, D, 10000.0)
    dq1, dk1, dv1 = ops.attn_bwd(q, k, v, out, lse, do, causal=True, rope_tables=(table, table))
    torch.cuda.synchronize()
    assert torch.equal(dv1, dv0)
    assert_parity(dq1, dq0.float(), 8e-3, "dq", seq_dim=1)     # the fused path rounds once, the other twice
    assert_parity(dk1, dk0.float(), 8e-3, "dk", seq_dim=1)
    with pytest.raises(Exception):
        ops.attn_bwd(q, k, v, out, lse, do, causal=True, dq=dq1, accumulate_dq=True, rope_tables=(table, table))


@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (4, 2)])
def test_attention_module_with_and_without_the_fused_rotation(Hq, Hkv, dev):
    """LlamaFlashAttention2TPSP forward and every gradient: fused node (projection + rotation + attention) against the
    chain of separate kernels and against the oracle."""
    import types
    from odysseus_transformer_amd.decoder.odysseus import LlamaFlashAttention2TPSP
    L, d, D = 512, 512, 128
    cfg = types.SimpleNamespace(hidden_size=d, num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D,
                                intermediate_size=1024, hidden_act="silu", attention_dropout=0.0, rms_norm_eps=1e-6,
                                rope_theta=10000.0, max_position_embeddings=1 << 20, pretraining_tp=1, num_hidden_layers=1)
    x = randn((1, L, d), 9500, dtype=torch.bfloat16)
    dy = randn((1, L, d), 9501, dtype=torch.bfloat16)
    w_qkv = randn(((Hq + 2 * Hkv) * D, d), 9502, std=0.05, dtype=torch.bfloat16)
    w_o = randn((d, Hq * D), 9503, std=0.05, dtype=torch.bfloat16)
    res = {}
    for fused in (True, False):
        attn = LlamaFlashAttention2TPSP(cfg, 0).to(torch.bfloat16).to(dev)
        attn.fuse_rope = fused
        with torch.no_grad():
            attn.qkv_proj.weight.copy_(w_qkv)
            attn.o_proj.weight.copy_(w_o)
        xg = x.to(dev).requires_grad_(True)

        def step():
            y = attn(xg, position_ids=torch.arange(L, device=dev)[None])[0]
            y.backward(dy.to(dev))
            return y
        y, names = _kernels_of(step)
        assert ("rope" in names) == (not fused), names
        assert ("gemm_bf16_nt_rope" in names) == fused, names
        res[fused] = [t.float().cpu() for t in (y, xg.grad, attn.qkv_proj.weight.grad, attn.o_proj.weight.grad)]
    # oracle: projection -> rotation -> attention -> projection, explicit backward
    pos = torch.arange(L)[None]
    qkv = oracle.linear_fwd(x.float(), w_qkv.float())
    q0, k0, v0 = oracle.split_qkv(qkv, Hq, Hkv, D)
    cos, sin = oracle.rope_cos_sin(pos, D, 10000.0, torch.float32)
    q, k = oracle.apply_rope(q0, cos, sin), oracle.apply_rope(k0, cos, sin)
    o, lse = oracle.attention_fwd(q, k, v0, causal=True)
    y_ref = oracle.linear_fwd(o.reshape(1, L, Hq * D), w_o.float())
    do2, dwo_ref, _ = oracle.linear_bwd(o.reshape(1, L, Hq * D), w_o.float(), dy.float())
    dq, dk, dv = oracle.attention_bwd(q, k, v0, o, lse, do2.view(1, L, Hq, D), causal=True)
    dqkv = torch.cat((oracle.apply_rope_bwd(dq, cos, sin), oracle.apply_rope_bwd(dk, cos, sin), dv), dim=2)
    dx_ref, dwqkv_ref, _ = oracle.linear_bwd(x.float(), w_qkv.float(), dqkv.reshape(1, L, -1))
    for fused in (True, False):
        for got, ref, what in zip(res[fused], (y_ref, dx_ref, dwqkv_ref, dwo_ref), ("y", "dx", "dWqkv", "dWo")):
            assert_parity(got, ref, TOL_BF16, f"fused={fused} {what}")


def test_rope_table_is_reused_for_the_same_position_tensor_only(dev):
    from odysseus_transformer_amd import ops
    pos = torch.arange(64, device=dev)[None]
    t1 = ops.rope_table(pos, 64, 128, 10000.0)
    assert ops.rope_table(pos, 64, 128, 10000.0) is t1                 # the next layer of the same forward pass
    assert ops.rope_table(pos, 64, 128, 500000.0) is not t1            # another base
    t3 = ops.rope_table(pos.clone(), 64, 128, 10000.0)                 # another tensor object
    assert t3 is not t1 and torch.equal(t3, t1)
    pos.add_(7)                                                        # modified in place: built again
    t4 = ops.rope_table(pos, 64, 128, 10000.0)
    assert ops.rope_table(pos, 64, 128, 10000.0) is t4 and not torch.equal(t4, t3)
