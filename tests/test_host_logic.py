"""CPU tests of the host side: slicing helpers, scratch arena, flatten rule, module
surface (names, shapes, constructor keywords, error behaviour).  No compute calls."""
import types

import pytest
import torch

from odysseus_transformer_amd import parallel_state as ps
from odysseus_transformer_amd.utils import apply_seq_parallel as asp
from odysseus_transformer_amd.utils import globals as g
from odysseus_transformer_amd.utils.comm import prepare_input_tensors_for_wgrad_compute


@pytest.fixture(autouse=True)
def _single_rank():
    ps.destroy_model_parallel()
    yield
    ps.destroy_model_parallel()


def _cfg(**kw):
    base = dict(hidden_size=64, num_attention_heads=8, num_key_value_heads=4, head_dim=8, intermediate_size=96,
                hidden_act="silu", attention_dropout=0.0, rms_norm_eps=1e-6, rope_theta=10000.0, pretraining_tp=1,
                num_hidden_layers=2)
    base.update(kw)
    return types.SimpleNamespace(**base)


# ------------------------------------------------------------------ prepare_attn_inputs
def test_prepare_attn_inputs_modes():
    L, N = 16, 4
    ids, pos, tgt = torch.arange(L)[None], torch.arange(L)[None], torch.arange(L)[None] + 100
    for r in range(N):
        o = asp.prepare_attn_inputs("odysseus", ids, pos, tgt, r, N, "cpu")
        assert o["local_input_ids"].tolist() == [list(range(4 * r, 4 * r + 4))]
        assert o["local_target_ids"].tolist() == [[100 + t for t in range(4 * r, 4 * r + 4)]]
        assert torch.equal(o["local_position_ids"], pos)                      # FULL position ids
        u = asp.prepare_attn_inputs("ulysses", ids, pos, tgt, r, N, "cpu")
        assert torch.equal(u["local_position_ids"], pos[:, 4 * r:4 * r + 4])
        t = asp.prepare_attn_inputs("tpsp", ids, pos, tgt, r, N, "cpu")
        assert all(torch.equal(t[k], o[k]) for k in o)
        z = asp.prepare_attn_inputs("ring", ids, pos, tgt, r, N, "cpu")
        assert z["local_input_ids"].tolist() == [[2 * r, 2 * r + 1, 2 * (2 * N - 1 - r), 2 * (2 * N - 1 - r) + 1]]
    d = asp.prepare_attn_inputs("dp", ids, pos, tgt, 1, N, "cpu")
    assert torch.equal(d["local_input_ids"], ids)
    assert asp.prepare_attn_inputs("odysseus", ids, pos, None, 0, N, "cpu")["local_target_ids"] is None
    with pytest.raises(ValueError, match="Invalid parallel_mode"):
        asp.prepare_attn_inputs("nope", ids, pos, tgt, 0, N, "cpu")
    # the shards of all ranks tile the sequence exactly once in every splitting mode
    for mode in ("odysseus", "ulysses", "ring"):
        got = torch.cat([asp.prepare_attn_inputs(mode, ids, pos, tgt, r, N, "cpu")["local_input_ids"] for r in range(N)], 1)
        assert sorted(got[0].tolist()) == list(range(L))


# ------------------------------------------------------------------ GlobalMemoryBuffer
def test_global_memory_buffer():
    g._destroy_global_memory_buffer()
    with pytest.raises(AssertionError):
        g.get_global_memory_buffer()
    g._set_global_memory_buffer("cpu")
    with pytest.raises(AssertionError):
        g._set_global_memory_buffer("cpu")
    buf = g.get_global_memory_buffer()
    a = buf.get_tensor([4, 8], torch.float32, "mpu")
    assert a.shape == (4, 8)
    b = buf.get_tensor([2, 8], torch.float32, "mpu")            # smaller request: same storage, no growth
    assert b.data_ptr() == a.data_ptr()
    c = buf.get_tensor([16, 8], torch.float32, "mpu")           # larger: grows
    assert c.numel() == 128 and buf.buffer[("mpu", torch.float32)].numel() == 128
    d = buf.get_tensor([4, 8], torch.bfloat16, "mpu")           # keyed by dtype as well
    assert d.dtype == torch.bfloat16 and d.data_ptr() != c.data_ptr()
    g._destroy_global_memory_buffer()


def test_wgrad_flatten_rule():
    dy = torch.randn(1, 6, 4).transpose(1, 2).transpose(1, 2)[:, :, ::1]
    dy_nc = torch.randn(1, 4, 6).transpose(1, 2)                # non-contiguous (1, 6, 4)
    x = torch.randn(1, 6, 5)
    g2, x2 = prepare_input_tensors_for_wgrad_compute(dy_nc, x)
    assert g2.shape == (6, 4) and x2.shape == (6, 5) and g2.is_contiguous()
    assert torch.equal(g2, dy_nc.reshape(6, 4))
    g3, x3 = prepare_input_tensors_for_wgrad_compute(dy_nc[0], x[0])   # 2-D passes through
    assert g3.shape == (6, 4) and x3.shape == (6, 5)


# ------------------------------------------------------------------ module surface
def test_attention_module_surface():
    from odysseus_transformer_amd.decoder.odysseus import LlamaFlashAttention2TPSP
    m = LlamaFlashAttention2TPSP(_cfg(), 3)
    assert m.layer_idx == 3 and m.pack_weight and m.sequence_parallel
    assert m.n_local_heads == 8 and m.n_local_kv_heads == 4
    assert m.q_proj is None and m.k_proj is None and m.v_proj is None
    assert {k: tuple(v.shape) for k, v in m.state_dict().items()} == {
        "qkv_proj.weight": ((8 + 2 * 4) * 8, 64), "o_proj.weight": (64, 64)}
    assert m.qkv_proj.bias is None and m.o_proj.bias is None
    u = LlamaFlashAttention2TPSP(_cfg(), 0, pack_weight=False, keep_master_weight_for_test=True)
    assert tuple(u.q_proj.weight.shape) == (64, 64) and tuple(u.k_proj.weight.shape) == (32, 64)
    assert u.q_proj.master_weight is not None
    with pytest.raises(AssertionError, match="bsz"):
        m(torch.zeros(2, 4, 64))
    with pytest.raises(RuntimeError, match="HIP device"):     # CPU tensors are refused: no fallback path
        m(torch.zeros(1, 4, 64))
    with pytest.raises(RuntimeError, match="HIP device"):     # a padding mask takes the general path, which needs the GPU too
        m(torch.zeros(1, 4, 64), attention_mask=torch.ones(1, 4))


def test_sharded_shapes_for_a_declared_group():
    """Parameter shapes follow the model-parallel layout exactly as in the reference:
    heads / N per rank, packed rows [q_local ; k_local ; v_local], row shards of the MLP."""
    from odysseus_transformer_amd.decoder.odysseus import LlamaFlashAttention2TPSP, LlamaMLPZeRO
    ps.initialize_model_parallel(4, rank=1)
    m = LlamaFlashAttention2TPSP(_cfg(), 0)
    assert m.n_local_heads == 2 and m.n_local_kv_heads == 1
    assert tuple(m.qkv_proj.weight.shape) == ((2 + 2 * 1) * 8, 64)
    assert tuple(m.o_proj.weight.shape) == (64, 16)
    mlp = LlamaMLPZeRO(_cfg())
    assert tuple(mlp.gate_up_proj.weight.shape) == (2 * 96 // 4, 64)
    assert tuple(mlp.down_proj.weight.shape) == (64 // 4, 96)
    with pytest.raises(AssertionError):
        ps.divide_and_check_no_remainder(10, 4)
    # collectives are outside this build: a forward on more than one rank says so
    with pytest.raises(NotImplementedError, match="outside this build"):
        from odysseus_transformer_amd.utils.linear_tpsp import _gather_along_first_dim
        _gather_along_first_dim(torch.zeros(1, 4, 64))


def test_partitioned_init_is_a_slice_of_one_master():
    from odysseus_transformer_amd.utils.linear_tpsp import ColumnParallelLinearAG, RowParallelLinearRS
    shards_c, shards_r = [], []
    for r in range(2):
        ps.initialize_model_parallel(2, rank=r)
        torch.manual_seed(0)
        c = ColumnParallelLinearAG(8, 12, bias=False, gather_output=False, keep_master_weight_for_test=True)
        torch.manual_seed(0)
        rr = RowParallelLinearRS(12, 8, bias=True, input_is_parallel=True, keep_master_weight_for_test=True)
        shards_c.append((c.weight.data, c.master_weight))
        shards_r.append((rr.weight.data, rr.master_weight))
        assert rr.bias is not None and tuple(rr.bias.shape) == (8,) and (rr.bias == 0).all()
    assert torch.equal(torch.cat([s[0] for s in shards_c], 0), shards_c[0][1])      # split along output rows
    assert torch.equal(torch.cat([s[0] for s in shards_r], 1), shards_r[0][1])      # split along input columns


def test_mlp_and_patcher_surface():
    from odysseus_transformer_amd.decoder.odysseus import (LlamaMLPZeRO, LlamaFlashAttention2TPSP,
                                                           apply_odysseus_attn_patch_llama)
    mlp = LlamaMLPZeRO(_cfg())
    assert tuple(mlp.gate_up_proj.weight.shape) == (192, 64) and tuple(mlp.down_proj.weight.shape) == (64, 96)
    with pytest.raises(NotImplementedError, match="pretraining_tp"):
        LlamaMLPZeRO(_cfg(pretraining_tp=2))(torch.zeros(1, 2, 64))
    transformers = pytest.importorskip("transformers")
    cfg = transformers.LlamaConfig(hidden_size=64, intermediate_size=96, num_hidden_layers=2, num_attention_heads=8,
                                   num_key_value_heads=4, vocab_size=50)
    model = transformers.LlamaForCausalLM(cfg).to(torch.bfloat16)
    apply_odysseus_attn_patch_llama(model, use_zero3_linear=False)
    assert isinstance(model.model.layers[1].self_attn, LlamaFlashAttention2TPSP)
    assert not isinstance(model.model.layers[1].mlp, LlamaMLPZeRO)
    apply_odysseus_attn_patch_llama(model)
    for layer in model.model.layers:
        assert isinstance(layer.mlp, LlamaMLPZeRO) and layer.self_attn.qkv_proj.weight.dtype == torch.bfloat16
        assert layer.self_attn.return_arity == 2        # this transformers unpacks two values


def test_functional_linear_signature_and_dead_branches():
    import inspect
    from odysseus_transformer_amd.utils import linear_tpsp as lt, linear_zero3 as lz
    assert list(inspect.signature(lt.linear_with_grad_accumulation_and_async_allreduce).parameters) == [
        "input", "weight", "bias", "gradient_accumulation_fusion", "async_grad_allreduce", "sequence_parallel",
        "grad_output_buffer"]
    assert list(inspect.signature(lz.linear_with_zero).parameters) == ["input", "weight", "bias"]
    assert list(inspect.signature(lz.LinearZeRO3.__init__).parameters) == ["self", "input_features",
                                                                           "output_features", "bias"]
    with pytest.raises(AssertionError, match="Batch size should be 1"):
        lt.linear_with_grad_accumulation_and_async_allreduce(torch.zeros(2, 3, 8), torch.zeros(4, 8), None, False,
                                                             False, True)


def test_bench_refuses_more_than_one_gpu():
    """One GPU only: `bench.py --gpus N` with N above 1 exits with a message that says so."""
    import subprocess
    import sys
    from pathlib import Path
    root = Path(__file__).resolve().parents[1]
    r = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


# ------------------------------------------------------------------ argument checks of the op wrappers
def test_rmsnorm_and_rope_wrappers_check_what_the_kernels_cannot():
    from odysseus_transformer_amd import ops
    x = torch.zeros(4, 16, dtype=torch.bfloat16)
    ops.check_rmsnorm_args(x, torch.ones(16, dtype=torch.bfloat16))
    with pytest.raises(TypeError, match="weight is torch.float32"):
        ops.check_rmsnorm_args(x, torch.ones(16))                      # fp32 weight, bf16 activations
    with pytest.raises(ValueError, match="weight must be"):
        ops.check_rmsnorm_args(x, torch.ones(8, dtype=torch.bfloat16))  # too short: the kernel would read past it
    with pytest.raises(ValueError, match="weight must be"):
        ops.check_rmsnorm_args(x, torch.ones(32, dtype=torch.bfloat16)[::2])
    with pytest.raises(ValueError, match="dy must match"):
        ops.check_rmsnorm_args(x, torch.ones(16, dtype=torch.bfloat16), torch.ones(4), torch.zeros(4, 16))
    with pytest.raises(ValueError, match="rstd must be"):
        ops.check_rmsnorm_args(x, torch.ones(16, dtype=torch.bfloat16), torch.ones(3), x)
    with pytest.raises(ValueError, match="rstd must be"):
        ops.check_rmsnorm_args(x, torch.ones(16, dtype=torch.bfloat16), torch.ones(4, dtype=torch.float64), x)
    q = torch.zeros(1, 8, 3, 16)
    ops.check_rope_args(q, 2, torch.arange(8)[None], torch.ones(8))
    with pytest.raises(ValueError, match="exceeds"):
        ops.check_rope_args(q, 4, None, None)
    with pytest.raises(ValueError, match="inv_freq must be"):
        ops.check_rope_args(q, 2, None, torch.ones(4))
    with pytest.raises(ValueError, match="inv_freq must be"):
        ops.check_rope_args(q, 2, None, torch.ones(8, dtype=torch.float64))
    with pytest.raises(ValueError, match="position_ids must be"):
        ops.check_rope_args(q, 2, torch.zeros(1, 8), None)
    with pytest.raises(ValueError, match="do not cover"):
        ops.check_rope_args(q, 2, torch.arange(7)[None], None)
    with pytest.raises(RuntimeError, match="only on a HIP device"):    # and no CPU fallback behind the checks
        ops.rmsnorm_fwd(x, torch.ones(16, dtype=torch.bfloat16))


def test_scratch_comes_from_the_arena_when_it_is_set_up():
    from odysseus_transformer_amd import ops
    g._destroy_global_memory_buffer()
    cpu = torch.device("cpu")
    a = ops.scratch(1000, "attn_fwd_workspace", cpu)
    b = ops.scratch(1000, "attn_fwd_workspace", cpu)
    assert a.data_ptr() != b.data_ptr() or a.data_ptr() == 0          # no arena: fresh allocations
    g._set_global_memory_buffer("cpu")
    try:
        a = ops.scratch(1000, "attn_fwd_workspace", cpu)
        b = ops.scratch(600, "attn_fwd_workspace", cpu)
        c = ops.scratch(600, "attn_bwd_workspace", cpu)
        assert a.data_ptr() == b.data_ptr() and c.data_ptr() != a.data_ptr()
        assert a.numel() == 1000 and b.numel() == 600 and a.dtype == torch.uint8
        big = ops.scratch(5000, "attn_fwd_workspace", cpu)                # grows, then stays
        assert ops.scratch(1000, "attn_fwd_workspace", cpu).data_ptr() == big.data_ptr()
        # an arena of another device type is not used
        assert ops.scratch(10, "x", torch.device("meta")).device.type == "meta"
    finally:
        g._destroy_global_memory_buffer()


def test_patchers_stop_the_host_from_building_dense_masks():
    """With attn_implementation='eager' transformers passes a dense causal mask to every layer,
    which the modules refuse; after the patch the forward reaches the ops (which refuse CPU tensors)."""
    transformers = pytest.importorskip("transformers")
    from odysseus_transformer_amd.decoder.odysseus import apply_odysseus_attn_patch_llama
    from odysseus_transformer_amd.decoder.tensor_parallel import LlamaMLPTPSP, apply_tpsp_attn_patch_llama
    for patch in (apply_odysseus_attn_patch_llama, apply_tpsp_attn_patch_llama):
        cfg = transformers.LlamaConfig(hidden_size=64, intermediate_size=96, num_hidden_layers=2, num_attention_heads=2,
                                       num_key_value_heads=1, head_dim=32, vocab_size=64)
        cfg._attn_implementation = "eager"
        model = transformers.LlamaForCausalLM(cfg)
        patch(model)
        assert model.config._attn_implementation == "flash_attention_2"
        with pytest.raises(RuntimeError, match="only on a HIP device"):
            model(torch.randint(0, 64, (1, 16)), position_ids=torch.arange(16)[None])
    assert isinstance(model.model.layers[0].mlp, LlamaMLPTPSP)
    assert tuple(model.model.layers[1].mlp.w1w3.weight.shape) == (192, 64)
    assert tuple(model.model.layers[1].mlp.w2.weight.shape) == (64, 96)


def test_tpsp_mlp_surface():
    from odysseus_transformer_amd.decoder.tensor_parallel import LlamaMLPTPSP
    from odysseus_transformer_amd.utils.linear_tpsp import ColumnParallelLinear, ColumnParallelLinearAG, RowParallelLinearRS
    m = LlamaMLPTPSP(_cfg())
    assert isinstance(m.w1w3, ColumnParallelLinearAG) and isinstance(m.w2, RowParallelLinearRS)
    assert m.w1w3.bias is None and m.w2.bias is None and m.w2.input_is_parallel
    m = LlamaMLPTPSP(_cfg(), pack_weight=True, sequence_parallel=False, keep_master_weight_for_test=True)
    assert type(m.w1w3) is ColumnParallelLinear and m.w1w3.master_weight is not None
    m = LlamaMLPTPSP(_cfg(), pack_weight=False)
    assert type(m.w1) is ColumnParallelLinear and tuple(m.w1.weight.shape) == (96, 64) and not hasattr(m, "w1w3")
    ps.initialize_model_parallel(4, 1)
    m = LlamaMLPTPSP(_cfg())
    assert tuple(m.w1w3.weight.shape) == (48, 64) and tuple(m.w2.weight.shape) == (64, 24)
    with pytest.raises(AssertionError, match="Pretraining TP"):
        LlamaMLPTPSP(_cfg(pretraining_tp=2))(torch.zeros(1, 4, 64))


def test_zigzag_step_table():
    """Which part of a received block a rank uses (zigzag ring): a source rank before it contributes its first
    chunk to all local queries, a source rank after it is seen by the second local chunk only."""
    from odysseus_transformer_amd.ops import ZigzagRingRankAttnFunc as Z
    assert Z._steps(0, 1) == [((0, 2), (0, 2), True)]
    # rank 1 of 4 receives the blocks of ranks 1, 0, 3, 2
    assert Z._steps(1, 4) == [((0, 2), (0, 2), True), ((0, 2), (0, 1), False), ((1, 2), (0, 2), False),
                              ((1, 2), (0, 2), False)]
    # brute force over token positions: the steps of every rank cover each (query, key <= query) chunk pair once
    for world in (1, 2, 3, 5):
        seen = {}
        for r in range(world):
            mine = (r, 2 * world - 1 - r)
            for s, ((q0, q1), (k0, k1), causal) in enumerate(Z._steps(r, world)):
                src = (r - s) % world
                theirs = (src, 2 * world - 1 - src)
                for qi in range(q0, q1):
                    for ki in range(k0, k1):
                        qc, kc = mine[qi], theirs[ki]
                        if causal and kc > qc:
                            continue            # masked inside the causal step
                        assert kc <= qc, (world, r, s, qc, kc)
                        seen[(qc, kc)] = seen.get((qc, kc), 0) + 1
        assert all(n == 1 for n in seen.values())
        assert len(seen) == (2 * world) * (2 * world + 1) // 2


def test_ring_and_ulysses_refuse_a_larger_world():
    import pytest as _pytest
    from odysseus_transformer_amd import parallel_state
    from odysseus_transformer_amd.decoder.ring import zigzag_ring_flash_attn_func
    from odysseus_transformer_amd.decoder.ulysses import ulysses_attn
    parallel_state.initialize_model_parallel(2, 0)
    try:
        with _pytest.raises(NotImplementedError):
            zigzag_ring_flash_attn_func(None, None, None, 0.0, None, causal=True)
        with _pytest.raises(NotImplementedError):
            ulysses_attn(None, None, None)
    finally:
        parallel_state.destroy_model_parallel()


def test_train_script_accepts_every_mode_of_the_reference():
    from odysseus_transformer_amd.train import parse_args
    for mode in ("odysseus", "ulysses", "dp", "tpsp", "ring"):
        assert parse_args(["--parallel_mode", mode]).parallel_mode == mode
    # every flag of the reference's parser (train.py:245-257) is accepted; the FSDP ones say what they do here
    ref_flags = ["--batch-size", "1", "--seed", "1", "--max-train-steps", "3", "--learning-rate", "1e-5", "--rope-theta", "1e4",
                 "--model", "x", "--seq-length", "1024", "--cpu-offload", "--grad-checkpoint", "--use_zero2", "--use_ody_zero3",
                 "--use_profiler", "--use_cfg_init_model"]
    a = parse_args(ref_flags)
    assert a.cpu_offload and a.use_zero2 and a.grad_checkpoint and a.use_profiler and a.seq_length == 1024
    from odysseus_transformer_amd.train import main
    with pytest.raises(NotImplementedError, match="cpu-offload"):
        main(a)


def test_adamw_host_side():
    """Hyper-parameter checks, the parameter-group keys that make its state dicts load into torch.optim.AdamW with the
    same meaning, and no CPU path."""
    import pytest as _pytest
    import torch
    from odysseus_transformer_amd.optim import AdamW
    with _pytest.raises(ValueError):
        AdamW([torch.nn.Parameter(torch.zeros(4))], betas=(1.0, 0.9))
    p = torch.nn.Parameter(torch.zeros(4))
    opt = AdamW([p], lr=1e-3)
    ref = torch.optim.AdamW([torch.nn.Parameter(torch.zeros(4))], lr=1e-3)
    assert set(ref.param_groups[0]) <= set(opt.param_groups[0])
    assert opt.param_groups[0]["decoupled_weight_decay"] is True
    opt.step()                                   # no gradient: nothing happens
    p.grad = torch.ones(4)
    with _pytest.raises(RuntimeError, match="no CPU implementation"):
        opt.step()


def test_general_attention_path_gathers_and_scatters_like_the_host(monkeypatch):
    """The host logic of the attention module's general path (padding mask, earlier cache content) on the CPU, with
    the kernel call replaced by the oracle's brute-force attention: masked tokens take part on neither side, the
    queries sit at the end of the keys, rows of masked queries are zero, a lone decoding query is always kept
    (decoder/odysseus.py:215-263 through the host's unpad / varlen / pad)."""
    import math
    from transformers import DynamicCache
    from oracle import odysseus_oracle as oracle
    from odysseus_transformer_amd import ops
    from odysseus_transformer_amd.decoder.odysseus import LlamaFlashAttention2TPSP
    seen = []

    def brute(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False, **kw):
        seen.append((q.shape[1], k.shape[1]))
        return oracle.attention_naive(q.double(), k.double(), v.double(), causal=causal, scale=softmax_scale)[0].to(q.dtype)
    monkeypatch.setattr(ops, "flash_attn_func", brute)
    m = LlamaFlashAttention2TPSP(_cfg(), 0)
    nh, nkv, D = m.n_local_heads, m.n_local_kv_heads, m.head_dim
    scale = 1.0 / math.sqrt(D)
    g = torch.Generator().manual_seed(5)

    def dense(q, k, v, mask):
        """every query row against all keys, with the mask and the positions written out"""
        Lq, Lk = q.shape[1], k.shape[1]
        kh = k.permute(0, 2, 1, 3).repeat_interleave(nh // nkv, dim=1).double()
        vh = v.permute(0, 2, 1, 3).repeat_interleave(nh // nkv, dim=1).double()
        s = torch.matmul(q.permute(0, 2, 1, 3).double(), kh.transpose(-1, -2)) * scale
        pos = torch.arange(Lq)[:, None] + (Lk - Lq)
        dead = (torch.arange(Lk)[None, :] > pos) | (mask[0] == 0)[None, :]
        o = torch.matmul(torch.softmax(s.masked_fill(dead, float("-inf")), dim=-1), vh).permute(0, 2, 1, 3)
        qdead = (mask[0, Lk - Lq:] == 0) if Lq > 1 else torch.zeros(1, dtype=torch.bool)
        return o.masked_fill(qdead[None, :, None, None], 0.0)

    # prefill with left padding and a hole in the middle
    L = 24
    q, k, v = torch.randn(1, L, nh, D, generator=g), torch.randn(1, L, nkv, D, generator=g), torch.randn(1, L, nkv, D, generator=g)
    mask = torch.ones(1, L, dtype=torch.long)
    mask[0, :5] = 0
    mask[0, 11:13] = 0
    y = m._attend_general(q, k, v, mask, None, None, scale)
    assert seen[-1] == (L - 7, L - 7)
    torch.testing.assert_close(y.double(), dense(q, k, v, mask), atol=1e-5, rtol=1e-5)
    assert torch.count_nonzero(y[0, :5]) == 0 and torch.count_nonzero(y[0, 11:13]) == 0
    # an all-ones mask and no mask are the plain call
    y1 = m._attend_general(q, k, v, torch.ones(1, L, dtype=torch.long), None, None, scale)
    y0 = m._attend_general(q, k, v, None, None, None, scale)
    assert torch.equal(y0, y1) and seen[-1] == (L, L)
    with pytest.raises(ValueError, match="padding mask"):
        m._attend_general(q, k, v, torch.ones(1, L + 1, dtype=torch.long), None, None, scale)
    # nothing kept: zeros, and no kernel call
    n = len(seen)
    assert torch.count_nonzero(m._attend_general(q, k, v, torch.zeros(1, L, dtype=torch.long), None, None, scale)) == 0
    assert len(seen) == n

    # earlier cache content: 6 new tokens behind the 24 cached ones, the prefill's padding still masked
    cache = DynamicCache()
    cache.update(k.transpose(1, 2), v.transpose(1, 2), 0, {})
    qn, kn, vn = torch.randn(1, 6, nh, D, generator=g), torch.randn(1, 6, nkv, D, generator=g), torch.randn(1, 6, nkv, D, generator=g)
    mask2 = torch.cat([mask, torch.ones(1, 6, dtype=torch.long)], dim=1)
    mask2[0, L + 2] = 0
    y = m._attend_general(qn, kn, vn, mask2, cache, torch.arange(L, L + 6), scale)
    assert cache.get_seq_length(0) == L + 6 and seen[-1] == (5, L + 6 - 8)
    k_all, v_all = torch.cat([k, kn], dim=1), torch.cat([v, vn], dim=1)
    torch.testing.assert_close(y.double(), dense(qn, k_all, v_all, mask2), atol=1e-5, rtol=1e-5)
    # one decoding token: kept whatever the mask says about it
    q1, k1, v1 = torch.randn(1, 1, nh, D, generator=g), torch.randn(1, 1, nkv, D, generator=g), torch.randn(1, 1, nkv, D, generator=g)
    mask3 = torch.cat([mask2, torch.ones(1, 1, dtype=torch.long)], dim=1)
    y = m._attend_general(q1, k1, v1, mask3, cache, torch.tensor([L + 6]), scale)
    assert seen[-1] == (1, L + 7 - 8)
    torch.testing.assert_close(y.double(), dense(q1, torch.cat([k_all, k1], 1), torch.cat([v_all, v1], 1), mask3), atol=1e-5, rtol=1e-5)
