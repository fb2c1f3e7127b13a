"""Zigzag ring attention, one rank at a time on one GPU: every rank's steps are run with the K/V blocks it
would receive over the ring (taken from the full tensors here), and the ranks' results, put back in global
order, must be the full causal attention of the oracle -- outputs, lse and every gradient."""
import pytest
import torch

from conftest import TOL_BF16, TOL_F32, TOL_LSE, assert_parity, randn, rel_err
import odysseus_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _kept_ds_budget():
    """Kept dS is opt-in; these tests opt in (a quarter of the device's memory, as the benchmark does) so that the
    full-size runs cover the kept-dS kernels.  The recomputing kernels are covered at full size by
    test_fullsize_gpu.py::test_cfg2_shard_whole_result and at small sizes by test_attention_gpu.py."""
    from odysseus_transformer_amd import ops
    ops.set_keep_ds_max_bytes(torch.cuda.get_device_properties(0).total_memory // 4)
    yield
    ops.set_keep_ds_max_bytes(None)


def _local(t, rank, world, dim=1):
    """Chunks r and 2N-1-r of the sequence (utils/apply_seq_parallel.py:93-99)."""
    ch = t.chunk(2 * world, dim=dim)
    return torch.cat([ch[rank], ch[2 * world - 1 - rank]], dim=dim)


def _scatter_add(full, local, rank, world, dim=1):
    c = local.shape[dim] // 2
    a, b = local.split(c, dim=dim)
    full.narrow(dim, rank * c, c).add_(a)
    full.narrow(dim, (2 * world - 1 - rank) * c, c).add_(b)


@pytest.mark.parametrize("world,c,Hq,Hkv,D,dtype", [(4, 96, 4, 2, 128, torch.bfloat16), (2, 160, 2, 2, 128, torch.bfloat16),
                                                   (3, 64, 4, 4, 64, torch.float32)])
def test_zigzag_ranks_assemble_to_full_causal_attention(world, c, Hq, Hkv, D, dtype, dev):
    from odysseus_transformer_amd import ops
    L = 2 * world * c
    q = randn((1, L, Hq, D), 8100, dtype=dtype)
    k = randn((1, L, Hkv, D), 8101, dtype=dtype)
    v = randn((1, L, Hkv, D), 8102, dtype=dtype)
    do = randn((1, L, Hq, D), 8103, dtype=dtype)
    o_ref, lse_ref = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=True)
    dq_ref, dk_ref, dv_ref = oracle.attention_bwd(q.float(), k.float(), v.float(), o_ref, lse_ref, do.float(), causal=True)

    out = torch.zeros((1, L, Hq, D)); lse = torch.zeros((1, Hq, L))
    dq = torch.zeros((1, L, Hq, D)); dk = torch.zeros((1, L, Hkv, D)); dv = torch.zeros((1, L, Hkv, D))
    for rank in range(world):
        print(f"zigzag world {world} rank {rank}", flush=True)
        ql = _local(q, rank, world).to(dev).requires_grad_(True)
        src = [(rank - s) % world for s in range(world)]
        ks = [_local(k, j, world).to(dev).requires_grad_(True) for j in src]
        vs = [_local(v, j, world).to(dev).requires_grad_(True) for j in src]
        o, l = ops.zigzag_ring_rank_attn(ql, ks, vs, rank, world)
        o.backward(_local(do, rank, world).to(dev))
        torch.cuda.synchronize()
        _scatter_add(out, o.detach().float().cpu(), rank, world)
        _scatter_add(lse, l.float().cpu(), rank, world, dim=2)
        _scatter_add(dq, ql.grad.float().cpu(), rank, world)
        for j, kk, vv in zip(src, ks, vs):     # a block's gradient belongs to the rank it came from
            _scatter_add(dk, kk.grad.float().cpu(), j, world)
            _scatter_add(dv, vv.grad.float().cpu(), j, world)
    tol = TOL_BF16 if dtype == torch.bfloat16 else TOL_F32
    assert_parity(out, o_ref, tol, "out", seq_dim=1)
    assert (lse - lse_ref).abs().max() <= TOL_LSE * max(1.0, lse_ref.abs().max().item())
    assert_parity(dq, dq_ref, tol, "dq", seq_dim=1)
    # dK / dV are sums of up to 2N bf16-rounded partial gradients (one per rank and step that read the chunk)
    gtol = 2 * tol if dtype == torch.bfloat16 else tol
    assert rel_err(dk, dk_ref) <= gtol, rel_err(dk, dk_ref)
    assert rel_err(dv, dv_ref) <= gtol, rel_err(dv, dv_ref)


def test_single_rank_ring_and_ulysses_are_the_flash_attention(dev):
    from odysseus_transformer_amd import ops
    from odysseus_transformer_amd.decoder.ring import zigzag_ring_flash_attn_func
    from odysseus_transformer_amd.decoder.ulysses import ulysses_attn
    q = randn((1, 300, 4, 128), 8200, dtype=torch.bfloat16).to(dev)
    k = randn((1, 300, 2, 128), 8201, dtype=torch.bfloat16).to(dev)
    v = randn((1, 300, 2, 128), 8202, dtype=torch.bfloat16).to(dev)
    ref = ops.flash_attn_func(q, k, v, 0.0, None, causal=True)
    assert torch.equal(zigzag_ring_flash_attn_func(q, k, v, 0.0, None, causal=True), ref)
    assert torch.equal(ulysses_attn(q, k, v, 0.0, None, causal=True), ref)
    # one rank, one step: the rank routine is the same causal attention
    o, _ = ops.zigzag_ring_rank_attn(q, [k], [v], 0, 1)
    assert rel_err(o, ref) <= 4e-3          # fp32 running pair rounded once vs. the kernel's own rounding
    with pytest.raises(NotImplementedError):
        zigzag_ring_flash_attn_func(q, k, v, 0.0, None, causal=False)


@pytest.mark.parametrize("mode", ["ulysses", "ring"])
def test_host_llama_with_attention_routed_to_the_hip_kernel(mode, dev):
    """The reference's monkey patches (decoder/ulysses.py:108-114, decoder/ring.py:98-104) on a small host
    model: logits and parameter gradients against the same model with the host's own eager attention in fp32."""
    transformers = pytest.importorskip("transformers")
    from transformers import LlamaConfig, LlamaForCausalLM
    from odysseus_transformer_amd.decoder.ring import apply_zigzag_ring_attn_monkey_patch_llama
    from odysseus_transformer_amd.decoder.ulysses import apply_ulysses_attn_monkey_patch_llama
    cfg = LlamaConfig(vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
                      num_key_value_heads=1, head_dim=128, max_position_embeddings=512, rms_norm_eps=1e-6, use_cache=False)
    cfg._attn_implementation = "eager"
    torch.manual_seed(0)
    ref_model = LlamaForCausalLM(cfg).float()
    ids = torch.randint(512, (1, 200), generator=torch.Generator().manual_seed(1))
    tgt = torch.randint(512, (200,), generator=torch.Generator().manual_seed(2))
    ref_logits = ref_model(ids, use_cache=False).logits
    torch.nn.functional.cross_entropy(ref_logits[0], tgt).backward()

    import copy
    model = copy.deepcopy(ref_model).to(torch.bfloat16).to(dev)
    model.zero_grad()
    (apply_ulysses_attn_monkey_patch_llama if mode == "ulysses" else apply_zigzag_ring_attn_monkey_patch_llama)(model)
    assert model.config._attn_implementation == "flash_attention_2"
    logits = model(ids.to(dev), position_ids=torch.arange(200, device=dev)[None], use_cache=False).logits
    torch.nn.functional.cross_entropy(logits[0].float(), tgt.to(dev)).backward()
    torch.cuda.synchronize()
    assert rel_err(logits, ref_logits.detach()) <= 3e-2     # a whole bf16 model against fp32
    g, g_ref = model.model.layers[0].self_attn.q_proj.weight.grad, ref_model.model.layers[0].self_attn.q_proj.weight.grad
    assert rel_err(g, g_ref) <= 5e-2
