"""GPU parity of the module layer: attention block, MLP and the whole decoder layer
(forward and every gradient) against the CPU oracle with the same seeded inputs."""
import types
import zlib

import pytest
import torch

from conftest import assert_parity, TOL_BF16, TOL_F32, TOL_LSE, randn, rel_err
import odysseus_oracle as oracle

pytestmark = pytest.mark.gpu


def _config(d, H, Hkv, D, i):
    return types.SimpleNamespace(hidden_size=d, num_attention_heads=H, num_key_value_heads=Hkv, head_dim=D,
                                 intermediate_size=i, hidden_act="silu", attention_dropout=0.0, rms_norm_eps=1e-6,
                                 rope_theta=10000.0, max_position_embeddings=1 << 20, pretraining_tp=1,
                                 num_hidden_layers=1)


def _params(d, H, Hkv, D, i, dtype, seed=0):
    p = {
        "ln1": 1.0 + randn((d,), seed + 1, std=0.02),
        "w_qkv": randn(((H + 2 * Hkv) * D, d), seed + 2, std=0.02),
        "w_o": randn((d, H * D), seed + 3, std=0.02),
        "ln2": 1.0 + randn((d,), seed + 4, std=0.02),
        "w_gate_up": randn((2 * i, d), seed + 5, std=0.02),
        "w_down": randn((d, i), seed + 6, std=0.02),
    }
    return {k: v.to(dtype) for k, v in p.items()}


def _load(layer, p, dev):
    layer = layer.to(dev)
    with torch.no_grad():
        layer.input_layernorm.weight.copy_(p["ln1"])
        layer.self_attn.qkv_proj.weight.copy_(p["w_qkv"])
        layer.self_attn.o_proj.weight.copy_(p["w_o"])
        layer.post_attention_layernorm.weight.copy_(p["ln2"])
        layer.mlp.gate_up_proj.weight.copy_(p["w_gate_up"])
        layer.mlp.down_proj.weight.copy_(p["w_down"])
    return layer


LAYER_CASES = [
    # name, L, d, H, Hkv, D, i, dtype
    ("cfg1_fp32", 2048, 512, 8, 8, 64, 1376, torch.float32),       # the reference's CPU-runnable configuration
    ("bf16_mha", 1024, 512, 4, 4, 128, 1408, torch.bfloat16),
    ("bf16_gqa_ragged", 520, 1024, 4, 1, 128, 2816, torch.bfloat16),
]


@pytest.mark.parametrize("case", LAYER_CASES, ids=lambda c: c[0])
def test_decoder_layer_fwd_bwd(case, dev):
    from odysseus_transformer_amd.decoder.odysseus import OdysseusDecoderLayer
    name, L, d, H, Hkv, D, i, dtype = case
    print(f"layer case {name}", flush=True)
    tol = TOL_BF16 if dtype == torch.bfloat16 else TOL_F32
    p = _params(d, H, Hkv, D, i, dtype)
    x = randn((1, L, d), 100, dtype=dtype)
    dy = randn((1, L, d), 101, dtype=dtype)
    pf = {k: v.float() for k, v in p.items()}
    y_ref, g_ref = oracle.decoder_layer_fwd_bwd(x.float(), pf, dy.float(), H, Hkv, D)

    layer = _load(OdysseusDecoderLayer(_config(d, H, Hkv, D, i)).to(dtype), p, dev)
    xg = x.to(dev).requires_grad_(True)
    pos = torch.arange(L, device=dev)[None]
    y = layer(xg, position_ids=pos)
    y.backward(dy.to(dev))
    torch.cuda.synchronize()
    assert_parity(y, y_ref, tol, f"{name} y")
    got = {
        "x": xg.grad, "ln1": layer.input_layernorm.weight.grad, "w_qkv": layer.self_attn.qkv_proj.weight.grad,
        "w_o": layer.self_attn.o_proj.weight.grad, "ln2": layer.post_attention_layernorm.weight.grad,
        "w_gate_up": layer.mlp.gate_up_proj.weight.grad, "w_down": layer.mlp.down_proj.weight.grad,
    }
    for k, v in got.items():
        assert_parity(v, g_ref[k], tol, f"{name} grad {k}")


def test_attention_block_unpacked_equals_packed(dev):
    """Three separate projections with rows [q ; k ; v] of the packed weight give the
    packed module's output (the identity the reference's tests rely on for w1w3)."""
    from odysseus_transformer_amd.decoder.odysseus import LlamaFlashAttention2TPSP
    d, H, Hkv, D, L = 512, 4, 2, 128, 384
    cfg = _config(d, H, Hkv, D, 1024)
    dt = torch.bfloat16
    packed = LlamaFlashAttention2TPSP(cfg, 0).to(dt).to(dev)
    unpacked = LlamaFlashAttention2TPSP(cfg, 0, pack_weight=False).to(dt).to(dev)
    w = randn(((H + 2 * Hkv) * D, d), 7, std=0.02, dtype=dt).to(dev)
    wo = randn((d, H * D), 8, std=0.02, dtype=dt).to(dev)
    with torch.no_grad():
        packed.qkv_proj.weight.copy_(w)
        packed.o_proj.weight.copy_(wo)
        unpacked.q_proj.weight.copy_(w[:H * D])
        unpacked.k_proj.weight.copy_(w[H * D:(H + Hkv) * D])
        unpacked.v_proj.weight.copy_(w[(H + Hkv) * D:])
        unpacked.o_proj.weight.copy_(wo)
    x = randn((1, L, d), 9, dtype=dt).to(dev)
    ya, none_a, cache_a = packed(x)
    yb = unpacked(x)[0]
    assert none_a is None and cache_a is None
    assert rel_err(ya, yb.float()) <= 1e-2
    y_ref, _ = oracle.attention_block(x.float().cpu(), w.float().cpu(), wo.float().cpu(), H, Hkv, D)
    assert rel_err(ya, y_ref) <= TOL_BF16


@pytest.mark.parametrize("fuse_layers", [False, True], ids=["modules_swapped", "layers_swapped"])
def test_patched_hf_llama_runs_and_matches_oracle(fuse_layers, dev):
    """apply_odysseus_attn_patch_llama on a small transformers Llama (attention and MLP modules swapped as in the
    reference, or whole decoder layers): logits and the gradient of the token embedding equal the oracle's
    composition of the same layers."""
    transformers = pytest.importorskip("transformers")
    from transformers import LlamaConfig, LlamaForCausalLM
    from odysseus_transformer_amd.decoder.odysseus import apply_odysseus_attn_patch_llama
    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
                      num_key_value_heads=1, head_dim=128, vocab_size=128, max_position_embeddings=2048,
                      rms_norm_eps=1e-6)
    model = LlamaForCausalLM(cfg).to(torch.bfloat16)
    apply_odysseus_attn_patch_llama(model, fuse_layers=fuse_layers)
    assert type(model.model.layers[0]).__name__ == ("OdysseusDecoderLayer" if fuse_layers else "LlamaDecoderLayer")
    with torch.no_grad():
        for n, prm in model.named_parameters():
            if "mlp" in n or "self_attn" in n:
                prm.copy_(randn(tuple(prm.shape), zlib.crc32(n.encode()) % 1000, std=0.02))
    model = model.to(dev)
    L = 200
    ids = torch.randint(0, 128, (1, L), generator=torch.Generator().manual_seed(1))
    pos = torch.arange(L)[None]
    logits = model(ids.to(dev), position_ids=pos.to(dev), use_cache=False).logits
    # oracle composition
    sd = {k: v.float().cpu() for k, v in model.state_dict().items()}
    h = sd["model.embed_tokens.weight"][ids]
    for l in range(2):
        pre = f"model.layers.{l}."
        p = {"ln1": sd[pre + "input_layernorm.weight"], "w_qkv": sd[pre + "self_attn.qkv_proj.weight"],
             "w_o": sd[pre + "self_attn.o_proj.weight"], "ln2": sd[pre + "post_attention_layernorm.weight"],
             "w_gate_up": sd[pre + "mlp.gate_up_proj.weight"], "w_down": sd[pre + "mlp.down_proj.weight"]}
        h = oracle.decoder_layer_fwd(h, p, 2, 1, 128)
    ref = oracle.linear_fwd(oracle.rmsnorm(h, sd["model.norm.weight"]), sd["lm_head.weight"])
    assert rel_err(logits, ref) <= TOL_BF16
    logits.float().square().mean().backward()
    assert model.model.layers[0].self_attn.qkv_proj.weight.grad is not None
    assert torch.isfinite(model.model.embed_tokens.weight.grad).all()


@pytest.mark.parametrize("case", [LAYER_CASES[0], LAYER_CASES[2]], ids=lambda c: c[0])
def test_layer_step_replayed_from_a_hip_graph(case, dev):
    """No entry point allocates, synchronises or clears memory with a memset, so a whole layer step
    (forward + backward) can be captured into a HIP graph.  Every replay -- with eager work and
    synchronisations in between -- must reproduce the eager result bit for bit."""
    from odysseus_transformer_amd.decoder.odysseus import OdysseusDecoderLayer
    name, L, d, H, Hkv, D, i, dtype = case
    print(f"graph case {name}", flush=True)
    layer = _load(OdysseusDecoderLayer(_config(d, H, Hkv, D, i)).to(dtype), _params(d, H, Hkv, D, i, dtype), dev)
    params = list(layer.parameters())
    x = randn((1, L, d), 31, dtype=dtype).to(dev).requires_grad_(True)
    dy = randn((1, L, d), 32, dtype=dtype).to(dev)
    pos = torch.arange(L, device=dev)[None]

    def step():
        for t in params + [x]:
            t.grad = None
        y = layer(x, position_ids=pos)
        y.backward(dy)
        return y

    side = torch.cuda.Stream()                      # warm-up off the default stream, as graph capture requires
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            y = step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    eager = [y.detach().clone(), x.grad.clone()] + [t.grad.clone() for t in params]
    del y                                           # drops the warm-up's autograd graph

    for t in params + [x]:
        t.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_g = layer(x, position_ids=pos)
        y_g.backward(dy)
    captured = [y_g.detach(), x.grad] + [t.grad for t in params]
    for replay in range(3):
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want), f"replay {replay} differs from the eager step"
        float(torch.randn(4096, device=dev).square().sum())   # eager work and a synchronisation between replays


def test_scratch_arena_removes_the_workspace_allocations(dev):
    """With the process-wide arena set up (utils/globals.py, as train.py:62 of the reference does),
    attention, split-K GEMM and RMSNorm scratch comes from its grow-only buffers: a layer step
    makes fewer allocator requests than without it, the buffers keep their addresses from step to
    step, and the results do not change."""
    from odysseus_transformer_amd.decoder.odysseus import OdysseusDecoderLayer
    from odysseus_transformer_amd.utils import globals as g
    name, L, d, H, Hkv, D, i, dtype = LAYER_CASES[1]
    layer = _load(OdysseusDecoderLayer(_config(d, H, Hkv, D, i)).to(dtype), _params(d, H, Hkv, D, i, dtype), dev)
    x = randn((1, L, d), 41, dtype=dtype).to(dev).requires_grad_(True)
    dy = randn((1, L, d), 42, dtype=dtype).to(dev)
    pos = torch.arange(L, device=dev)[None]

    def step():
        for t in list(layer.parameters()) + [x]:
            t.grad = None
        y = layer(x, position_ids=pos)
        y.backward(dy)
        torch.cuda.synchronize()
        return [y.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in layer.parameters()]

    def counted(fn):
        a0 = torch.cuda.memory_stats()["allocation.all.allocated"]
        out = fn()
        return out, torch.cuda.memory_stats()["allocation.all.allocated"] - a0

    g._destroy_global_memory_buffer()
    step()
    plain, n_plain = counted(step)
    g._set_global_memory_buffer(dev)
    try:
        step()                                       # the arena grows to its steady size here
        ptrs = {k: v.data_ptr() for k, v in g.get_global_memory_buffer().buffer.items()}
        assert {k[0] for k in ptrs} >= {"attn_fwd_workspace", "attn_bwd_workspace", "rmsnorm_dw_partials"}
        with_arena, n_arena = counted(step)
        _, n_arena2 = counted(step)
        assert {k: v.data_ptr() for k, v in g.get_global_memory_buffer().buffer.items()} == ptrs
        assert n_arena == n_arena2 and n_arena <= n_plain - 4, (n_plain, n_arena)   # fwd ws, bwd ws, 2 x norm partials
        for a, b in zip(plain, with_arena):
            assert torch.equal(a, b)
    finally:
        g._destroy_global_memory_buffer()


def test_linears_follow_autocast(dev):
    """fp32 modules under torch.autocast(bfloat16): the products run in bf16 as torch.matmul would
    (the reference's custom_fwd / custom_bwd, utils/linear_tpsp.py:129,180), outputs are bf16 and
    the weight gradients arrive in the parameters' fp32."""
    from odysseus_transformer_amd.utils.linear_tpsp import ColumnParallelLinearAG, RowParallelLinearRS
    from odysseus_transformer_amd.utils.linear_zero3 import LinearZeRO3
    x = randn((1, 256, 512), 51).to(dev).requires_grad_(True)
    w = randn((768, 512), 52, std=0.02)
    for make in (lambda: ColumnParallelLinearAG(512, 768, bias=False, gather_output=False),
                 lambda: RowParallelLinearRS(512, 768, bias=False, input_is_parallel=True),
                 lambda: LinearZeRO3(512, 768)):
        m = make().to(dev)
        with torch.no_grad():
            m.weight.copy_(w)
        x.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = m(x)
        assert y.dtype == torch.bfloat16
        y.float().sum().backward()
        assert m.weight.grad.dtype == torch.float32 and x.grad.dtype == torch.float32
        y_ref = oracle.linear_fwd(x.detach().cpu().bfloat16().float(), w.bfloat16().float())
        assert rel_err(y, y_ref) <= TOL_BF16
        assert rel_err(m.weight.grad, x.detach().cpu()[0].sum(0)[None].expand(768, 512)) <= TOL_BF16
        with pytest.raises(TypeError):               # outside autocast a dtype mismatch still raises
            m(x.bfloat16())


def test_fused_attention_under_inference_mode_and_with_hooks(dev):
    """The fused projection -> rotary -> attention node must work on position ids created under
    torch.inference_mode() (such tensors carry no version counter), and a forward hook registered on a projection
    must still run: its presence sends the call down the module-by-module path, with the same result."""
    from odysseus_transformer_amd.decoder.odysseus import LlamaFlashAttention2TPSP
    d, H, Hkv, D, L = 512, 4, 2, 128, 320
    attn = LlamaFlashAttention2TPSP(_config(d, H, Hkv, D, 1024), 0).to(torch.bfloat16).to(dev)
    attn.fuse_rope = True
    with torch.no_grad():
        attn.qkv_proj.weight.copy_(randn(((H + 2 * Hkv) * D, d), 41, std=0.02))
        attn.o_proj.weight.copy_(randn((d, H * D), 42, std=0.02))
    x = randn((1, L, d), 43, dtype=torch.bfloat16).to(dev)
    y_ref, _ = oracle.attention_block(x.float().cpu(), attn.qkv_proj.weight.float().cpu(), attn.o_proj.weight.float().cpu(),
                                      H, Hkv, D)
    with torch.inference_mode():
        pos = torch.arange(L, device=dev)[None]
        y1 = attn(x, position_ids=pos)[0]
        y2 = attn(x, position_ids=pos)[0]            # second layer call with the same position tensor: the cached table
    assert torch.equal(y1, y2)
    assert rel_err(y1, y_ref) <= TOL_BF16
    seen = []
    handle = attn.qkv_proj.register_forward_hook(lambda mod, args, out: seen.append(tuple(out.shape)))
    try:
        y3 = attn(x, position_ids=torch.arange(L, device=dev)[None])[0]
    finally:
        handle.remove()
    assert seen == [(1, L, (H + 2 * Hkv) * D)], "the hook on qkv_proj did not run"
    assert rel_err(y3, y_ref) <= TOL_BF16 and rel_err(y3, y1.float()) <= 1e-2


def test_zigzag_ring_patch_on_a_mistral_host(dev):
    """apply_zigzag_ring_attn_patch_mistral (decoder/ring.py:107-113): a small transformers Mistral whose attention
    goes through the HIP kernel gives the logits of the same model with the host's own eager attention in fp32."""
    transformers = pytest.importorskip("transformers")
    from transformers import MistralConfig, MistralForCausalLM
    from odysseus_transformer_amd.decoder.ring import apply_zigzag_ring_attn_patch_mistral, apply_zigzag_ring_attn_patch_llama
    assert callable(apply_zigzag_ring_attn_patch_llama)
    torch.manual_seed(0)
    cfg = MistralConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
                        num_key_value_heads=1, head_dim=128, vocab_size=128, max_position_embeddings=2048,
                        sliding_window=None, rms_norm_eps=1e-6)
    cfg._attn_implementation = "eager"
    host = MistralForCausalLM(cfg)
    L = 300
    ids = torch.randint(0, 128, (1, L), generator=torch.Generator().manual_seed(2))
    pos = torch.arange(L)[None]
    with torch.no_grad():
        ref = host(ids, position_ids=pos, use_cache=False).logits.float()
    model = MistralForCausalLM(cfg)
    model.load_state_dict(host.state_dict())
    model = model.to(torch.bfloat16).to(dev)
    apply_zigzag_ring_attn_patch_mistral(model)
    assert model.config._attn_implementation == "flash_attention_2"
    with torch.no_grad():
        logits = model(ids.to(dev), position_ids=pos.to(dev), use_cache=False).logits
    # bf16 weights and activations against the fp32 host: the bar of a whole bf16 model, not of one kernel
    assert rel_err(logits, ref) <= 5e-2


@pytest.mark.parametrize("pack_weight", [True, False], ids=["packed", "unpacked"])
def test_attention_block_with_a_padding_mask(pack_weight, dev):
    """A (1, L) padding mask (decoder/odysseus.py:256-263 hands it to the host's flash-attention forward, which
    drops the masked tokens, attends over the rest and pads the result with zeros): the kept tokens get what the
    oracle computes on the kept tokens alone, at their own positions; masked tokens get zero rows and send no
    gradient anywhere."""
    from odysseus_transformer_amd.decoder.odysseus import LlamaFlashAttention2TPSP
    d, H, Hkv, D, L = 512, 4, 2, 128, 300
    dt = torch.bfloat16
    attn = LlamaFlashAttention2TPSP(_config(d, H, Hkv, D, 1024), 0, pack_weight=pack_weight).to(dt).to(dev)
    w = randn(((H + 2 * Hkv) * D, d), 17, std=0.02, dtype=dt)
    wo = randn((d, H * D), 18, std=0.02, dtype=dt)
    with torch.no_grad():
        if pack_weight:
            attn.qkv_proj.weight.copy_(w)
        else:
            attn.q_proj.weight.copy_(w[:H * D])
            attn.k_proj.weight.copy_(w[H * D:(H + Hkv) * D])
            attn.v_proj.weight.copy_(w[(H + Hkv) * D:])
        attn.o_proj.weight.copy_(wo)
    x = randn((1, L, d), 19, dtype=dt)
    mask = torch.ones(1, L, dtype=torch.long)
    mask[0, :37] = 0          # left padding
    mask[0, 150:161] = 0      # and a hole
    keep = mask[0].nonzero().squeeze(1)
    pos = (mask.cumsum(1) - 1).clamp(min=0)       # the positions a host derives from the mask
    xg = x.to(dev).requires_grad_(True)
    y = attn(xg, attention_mask=mask.to(dev), position_ids=pos.to(dev))[0]
    dy = randn((1, L, d), 20, dtype=dt)
    y.backward(dy.to(dev))
    xr = x.float()[:, keep].requires_grad_(True)
    y_ref, _ = oracle.attention_block(xr, w.float(), wo.float(), H, Hkv, D, position_ids=pos[:, keep], differentiable=True)
    y_ref.backward(dy.float()[:, keep])
    assert_parity(y[:, keep.to(dev)], y_ref.detach(), TOL_BF16, "kept rows")
    gone = (mask[0] == 0).nonzero().squeeze(1).to(dev)
    assert torch.count_nonzero(y[:, gone]) == 0 and torch.count_nonzero(xg.grad[:, gone]) == 0
    assert_parity(xg.grad[:, keep.to(dev)], xr.grad, TOL_BF16, "dx of the kept rows", 1e-3)
    # a mask without zeros is the unmasked call
    y_all = attn(xg.detach(), attention_mask=torch.ones(1, L, dtype=torch.long, device=dev))[0]
    assert torch.equal(y_all, attn(xg.detach())[0])
    with pytest.raises(ValueError):
        attn(xg.detach(), attention_mask=torch.ones(1, L + 1, dtype=torch.long, device=dev))


def test_attention_block_decodes_from_a_kv_cache(dev):
    """Prefill into the host's DynamicCache, then more tokens against the cached keys (decoder/odysseus.py:215-220):
    every step gives the rows that the oracle computes for the whole sequence at once."""
    from transformers import DynamicCache
    from odysseus_transformer_amd.decoder.odysseus import LlamaFlashAttention2TPSP
    d, H, Hkv, D, L0 = 512, 4, 2, 128, 200
    dt = torch.bfloat16
    attn = LlamaFlashAttention2TPSP(_config(d, H, Hkv, D, 1024), 0).to(dt).to(dev).eval()
    w = randn(((H + 2 * Hkv) * D, d), 27, std=0.02, dtype=dt)
    wo = randn((d, H * D), 28, std=0.02, dtype=dt)
    with torch.no_grad():
        attn.qkv_proj.weight.copy_(w)
        attn.o_proj.weight.copy_(wo)
    steps = [L0, 1, 1, 7, 1]                      # prefill, single tokens, a chunk of 7
    L = sum(steps)
    x = randn((1, L, d), 29, dtype=dt)
    y_ref, _ = oracle.attention_block(x.float(), w.float(), wo.float(), H, Hkv, D)
    cache = DynamicCache()
    at = 0
    with torch.no_grad():
        for n in steps:
            pos = torch.arange(at, at + n, device=dev)[None]
            y, _, c = attn(x[:, at:at + n].to(dev), position_ids=pos, past_key_value=cache, use_cache=True, cache_position=pos[0])
            assert c is cache and cache.get_seq_length(0) == at + n
            assert_parity(y, y_ref[:, at:at + n], TOL_BF16, f"rows {at}..{at + n}", 1e-3)
            at += n
    # with a padding mask over cached and new keys: the masked cache entries take no part
    mask = torch.ones(1, L + 1, dtype=torch.long)
    mask[0, :5] = 0
    xn = randn((1, 1, d), 30, dtype=dt)
    pos = torch.tensor([[L - 5]], device=dev)
    with torch.no_grad():
        y = attn(xn.to(dev), attention_mask=mask.to(dev), position_ids=pos, past_key_value=cache, use_cache=True)[0]
    # oracle: the kept tokens 5..L-1 at positions 5..L-1 as they were cached, the new one at position L - 5
    xs = torch.cat([x.float()[:, 5:], xn.float()], 1)
    ps = torch.cat([torch.arange(5, L), torch.tensor([L - 5])])[None]
    y2, _ = oracle.attention_block(xs, w.float(), wo.float(), H, Hkv, D, position_ids=ps)
    assert_parity(y, y2[:, -1:], TOL_BF16, "masked decode step", 1e-3)


def test_attention_block_trains_with_attention_dropout(dev):
    """config.attention_dropout > 0 (decoder/odysseus.py:228 passes it on while training): the module drops entries
    of P with a seed it draws from torch's generator, and eval mode does not drop."""
    from odysseus_transformer_amd.decoder.odysseus import LlamaFlashAttention2TPSP
    d, H, Hkv, D, L = 512, 4, 2, 128, 320
    dt = torch.bfloat16
    cfg = _config(d, H, Hkv, D, 1024)
    cfg.attention_dropout = 0.25
    attn = LlamaFlashAttention2TPSP(cfg, 0).to(dt).to(dev)
    w = randn(((H + 2 * Hkv) * D, d), 37, std=0.02, dtype=dt)
    wo = randn((d, H * D), 38, std=0.02, dtype=dt)
    with torch.no_grad():
        attn.qkv_proj.weight.copy_(w)
        attn.o_proj.weight.copy_(wo)
    x = randn((1, L, d), 39, dtype=dt)
    attn.eval()
    y_eval = attn(x.to(dev))[0]
    y_ref, _ = oracle.attention_block(x.float(), w.float(), wo.float(), H, Hkv, D)
    assert_parity(y_eval, y_ref, TOL_BF16, "eval mode: no dropout")
    attn.train()
    torch.manual_seed(5)
    seed = int(torch.randint(0, 1 << 62, (1,)).item())
    torch.manual_seed(5)
    xg = x.to(dev).requires_grad_(True)
    y = attn(xg)[0]
    dy = randn((1, L, d), 40, dtype=dt)
    y.backward(dy.to(dev))
    # the oracle's block with the same mask
    xr = x.float().requires_grad_(True)
    qr, kr, vr = oracle.split_qkv(oracle.linear_fwd(xr, w.float()), H, Hkv, D)
    cos, sin = oracle.rope_cos_sin(torch.arange(L)[None], D, 10000.0, torch.float32)
    qr, kr = oracle.apply_rope(qr, cos, sin), oracle.apply_rope(kr, cos, sin)
    keep = oracle.dropout_keep_mask(seed, 0.25, 1, H, torch.arange(L), torch.arange(L))
    o, _ = oracle.attention_naive(qr, kr, vr, causal=True, keep=keep, dropout_p=0.25)
    yr = oracle.linear_fwd(o.reshape(1, L, H * D), wo.float())
    yr.backward(dy.float())
    assert_parity(y, yr.detach(), TOL_BF16, "training mode: dropped")
    assert rel_err(y, y_eval.float().cpu()) > 0.05
    assert_parity(xg.grad, xr.grad, TOL_BF16, "dx", 1e-3)
