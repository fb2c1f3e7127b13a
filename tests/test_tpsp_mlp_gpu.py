"""The TP-SP MLP (decoder/tensor_parallel.py of the reference) on one GPU, with the identities the
reference's own test asserts (tests/mlp_test.py:46-88): packed == unpacked (w1 = w1w3[:blk],
w3 = w1w3[blk:]) == packed with the sequence-parallel linear == ZeRO-3 MLP in the forward, and the
packed weight gradient agrees between the two packed variants -- plus parity with the oracle."""
import types

import pytest
import torch

from conftest import TOL_BF16, assert_parity, randn, rel_err
import odysseus_oracle as oracle

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _cfg(d, i):
    return types.SimpleNamespace(hidden_size=d, intermediate_size=i, hidden_act="silu", pretraining_tp=1,
                                 num_attention_heads=8, num_key_value_heads=8, num_hidden_layers=2)


@pytest.mark.parametrize("d,i,T", [(512, 2048, 32), (4096, 11008, 8192)], ids=["reference_test_shape", "llama7b_8k"])
def test_mlp_variants_agree_and_match_the_oracle(d, i, T, dev):
    from odysseus_transformer_amd.decoder.odysseus import LlamaMLPZeRO
    from odysseus_transformer_amd.decoder.tensor_parallel import LlamaMLPTPSP
    print(f"TP-SP MLP d={d} i={i} T={T}", flush=True)
    cfg = _cfg(d, i)
    x = randn((1, T, d), 1, dtype=BF).to(dev)
    dy = randn((1, T, d), 2, dtype=BF).to(dev)
    w13 = randn((2 * i, d), 3, std=0.02, dtype=BF)
    w2 = randn((d, i), 4, std=0.02, dtype=BF)

    m1 = LlamaMLPTPSP(cfg, pack_weight=True, sequence_parallel=False, keep_master_weight_for_test=True).to(BF).to(dev)
    m2 = LlamaMLPTPSP(cfg, pack_weight=False).to(BF).to(dev)
    m3 = LlamaMLPTPSP(cfg, pack_weight=True, sequence_parallel=True).to(BF).to(dev)
    m4 = LlamaMLPZeRO(cfg).to(BF).to(dev)
    with torch.no_grad():
        m1.w1w3.weight.copy_(w13)
        m1.w2.weight.copy_(w2)
        m2.w2.weight.copy_(m1.w2.weight)
        m2.w1.weight.copy_(m1.w1w3.weight[:i])
        m2.w3.weight.copy_(m1.w1w3.weight[i:])
        m3.w2.weight.copy_(m1.w2.weight)
        m3.w1w3.weight.copy_(m1.w1w3.weight)
        # ZeRO-3: the shard is a row block of the full weights rebuilt from the unpacked module's masters
        m4.gate_up_proj.weight.copy_(torch.cat([m2.w1.get_master_weight(), m2.w3.get_master_weight()], 0))
        m4.down_proj.weight.copy_(m2.w2.get_master_weight())
    outs, xs = [], []
    for m in (m1, m2, m3, m4):
        xi = x.clone().requires_grad_(True)
        o = m(xi)
        o.backward(dy)
        outs.append(o)
        xs.append(xi.grad)
    torch.cuda.synchronize()
    o1, o2, o3, o4 = outs
    # the reference asserts allclose with atol 1e-1 / rtol 1e-3; the same kernels run here, so the
    # packed variants agree bit for bit and the unpacked one too (same products, same SwiGLU)
    assert torch.equal(o1, o3) and torch.equal(o1, o4) and torch.equal(o1, o2)
    assert torch.equal(m1.w1w3.weight.grad, m3.w1w3.weight.grad)
    assert torch.equal(m1.w1w3.weight.grad, m4.gate_up_proj.weight.grad)
    assert torch.equal(torch.cat([m2.w1.weight.grad, m2.w3.weight.grad], 0), m1.w1w3.weight.grad)
    assert torch.equal(m1.w2.weight.grad, m2.w2.weight.grad)
    assert torch.equal(xs[0], xs[2]) and torch.equal(xs[0], xs[3])
    # the unpacked module's dx is the sum of two separately rounded products
    assert rel_err(xs[1], xs[0].float()) <= 1e-2
    # and against the oracle
    xf, dyf = x.float().cpu(), dy.float().cpu()
    y_ref = oracle.swiglu_mlp_fwd(xf, w13.float(), w2.float())
    dx_ref, dw13_ref, dw2_ref = oracle.swiglu_mlp_bwd(xf, w13.float(), w2.float(), dyf)
    assert_parity(o1, y_ref, TOL_BF16, "y")
    assert_parity(xs[0], dx_ref, TOL_BF16, "dx")
    assert_parity(m1.w1w3.weight.grad, dw13_ref, TOL_BF16, "dW13")
    assert_parity(m1.w2.weight.grad, dw2_ref, TOL_BF16, "dW2")


def test_tpsp_patch_swaps_modules(dev):
    transformers = pytest.importorskip("transformers")
    from odysseus_transformer_amd.decoder.odysseus import LlamaFlashAttention2TPSP
    from odysseus_transformer_amd.decoder.tensor_parallel import LlamaMLPTPSP, apply_tpsp_attn_patch_llama
    cfg = transformers.LlamaConfig(hidden_size=256, intermediate_size=512, num_attention_heads=2, num_key_value_heads=1,
                                   num_hidden_layers=2, vocab_size=128, head_dim=128)
    cfg._attn_implementation = "eager"          # the patcher makes the host stop building dense masks
    model = transformers.LlamaForCausalLM(cfg).to(BF)
    apply_tpsp_attn_patch_llama(model)
    for layer in model.model.layers:
        assert isinstance(layer.self_attn, LlamaFlashAttention2TPSP) and isinstance(layer.mlp, LlamaMLPTPSP)
    model = model.to(dev)
    ids = torch.randint(0, 128, (1, 96), generator=torch.Generator().manual_seed(0)).to(dev)
    logits = model(ids, position_ids=torch.arange(96, device=dev)[None]).logits
    loss = logits.float().logsumexp(-1).mean()
    loss.backward()
    assert torch.isfinite(logits).all()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters())
