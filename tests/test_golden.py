"""The committed vectors of tests/golden (made by tests/golden/make_golden.py from the installed
transformers' LlamaDecoderLayer and torch's SDPA in fp64, both independent of the oracle):
the CPU oracle must reproduce them, and so must the HIP path in fp32."""
from pathlib import Path

import numpy as np
import pytest
import torch

from conftest import TOL_F32, TOL_LSE, rel_err
import odysseus_oracle as oracle

GOLD = np.load(Path(__file__).resolve().parent / "golden" / "llama_layer_small.npz")
PARAMS = ("ln1", "w_qkv", "w_o", "ln2", "w_gate_up", "w_down")


def t(name):
    return torch.from_numpy(GOLD[name])


def test_oracle_reproduces_the_golden_layer():
    H, Hkv, D, d, i, L = (int(v) for v in GOLD["layer_dims"])
    p = {k: t(f"layer_p_{k}").double() for k in PARAMS}
    y, g = oracle.decoder_layer_fwd_bwd(t("layer_x").double(), p, t("layer_dy").double(), H, Hkv, D)
    assert rel_err(y, t("layer_y")) <= 1e-5
    for k in PARAMS + ("x",):
        assert rel_err(g[k], t(f"layer_g_{k}")) <= 1e-5, k


def test_oracle_reproduces_the_golden_attention():
    q, k, v, do = (t(f"attn_{n}").double() for n in ("q", "k", "v", "do"))
    o, lse = oracle.attention_fwd(q, k, v, causal=True)
    dq, dk, dv = oracle.attention_bwd(q, k, v, o, lse, do, causal=True)
    assert rel_err(o, t("attn_o")) <= 1e-6 and torch.allclose(lse.float(), t("attn_lse"), atol=1e-5)
    assert rel_err(dq, t("attn_dq")) <= 1e-6 and rel_err(dk, t("attn_dk")) <= 1e-6 and rel_err(dv, t("attn_dv")) <= 1e-6


@pytest.mark.gpu
def test_hip_layer_reproduces_the_golden_layer(dev):
    from odysseus_transformer_amd.decoder.odysseus import OdysseusDecoderLayer
    from test_layer_gpu import _config, _load
    H, Hkv, D, d, i, L = (int(v) for v in GOLD["layer_dims"])
    p = {k: t(f"layer_p_{k}") for k in PARAMS}
    layer = _load(OdysseusDecoderLayer(_config(d, H, Hkv, D, i)).to(torch.float32), p, dev)
    x = t("layer_x").to(dev).requires_grad_(True)
    y = layer(x, position_ids=torch.arange(L, device=dev)[None])
    y.backward(t("layer_dy").to(dev))
    assert rel_err(y, t("layer_y")) <= TOL_F32
    got = {"x": x.grad, "ln1": layer.input_layernorm.weight.grad, "w_qkv": layer.self_attn.qkv_proj.weight.grad,
           "w_o": layer.self_attn.o_proj.weight.grad, "ln2": layer.post_attention_layernorm.weight.grad,
           "w_gate_up": layer.mlp.gate_up_proj.weight.grad, "w_down": layer.mlp.down_proj.weight.grad}
    for k, v in got.items():
        assert rel_err(v, t(f"layer_g_{k}")) <= TOL_F32, k


@pytest.mark.gpu
def test_hip_attention_reproduces_the_golden_attention(dev):
    from odysseus_transformer_amd import ops
    q, k, v, do = (t(f"attn_{n}").to(dev) for n in ("q", "k", "v", "do"))
    o, lse = ops.attn_fwd(q, k, v, causal=True)
    dq, dk, dv = ops.attn_bwd(q, k, v, o, lse, do, causal=True)
    assert rel_err(o, t("attn_o")) <= TOL_F32
    assert torch.allclose(lse.cpu(), t("attn_lse"), atol=TOL_LSE, rtol=TOL_LSE)
    assert rel_err(dq, t("attn_dq")) <= TOL_F32 and rel_err(dk, t("attn_dk")) <= TOL_F32
    assert rel_err(dv, t("attn_dv")) <= TOL_F32


# ---------------------------------------------------------------------------------------------
# head_dim 128 (the bf16 MFMA kernels behind the benchmark numbers): GQA 2:1, 300 / 260 tokens, i.e.
# more than one 256-query block with a ragged last tile; the inputs are exact in bfloat16
# ---------------------------------------------------------------------------------------------
GOLD128 = np.load(Path(__file__).resolve().parent / "golden" / "llama_d128.npz")


def t128(name):
    if name + "_bf16bits" in GOLD128:
        return torch.from_numpy(GOLD128[name + "_bf16bits"]).view(torch.bfloat16)
    return torch.from_numpy(GOLD128[name])


def test_oracle_reproduces_the_golden_head_dim_128_vectors():
    H, Hkv, D, d, i, L = (int(v) for v in GOLD128["layer_dims"])
    assert (D, Hkv, L) == (128, 1, 260)
    p = {k: t128(f"layer_p_{k}").double() for k in PARAMS}
    y, g = oracle.decoder_layer_fwd_bwd(t128("layer_x").double(), p, t128("layer_dy").double(), H, Hkv, D)
    assert rel_err(y, t128("layer_y")) <= 1e-5
    for k in PARAMS + ("x",):
        assert rel_err(g[k], t128(f"layer_g_{k}")) <= 1e-5, k
    q, k, v, do = (t128(f"attn_{n}").double() for n in ("q", "k", "v", "do"))
    o, lse = oracle.attention_fwd(q, k, v, causal=True)
    dq, dk, dv = oracle.attention_bwd(q, k, v, o, lse, do, causal=True)
    assert rel_err(o, t128("attn_o")) <= 1e-6 and torch.allclose(lse.float(), t128("attn_lse"), atol=1e-5)
    for a, n in ((dq, "dq"), (dk, "dk"), (dv, "dv")):
        assert rel_err(a, t128(f"attn_{n}")) <= 1e-6, n


@pytest.mark.gpu
def test_hip_bf16_kernels_reproduce_the_golden_head_dim_128_vectors(dev):
    from conftest import TOL_BF16, assert_parity
    from odysseus_transformer_amd import ops
    from odysseus_transformer_amd.decoder.odysseus import OdysseusDecoderLayer
    from test_layer_gpu import _config, _load
    q, k, v, do = (t128(f"attn_{n}").to(dev) for n in ("q", "k", "v", "do"))
    assert q.dtype == torch.bfloat16 and q.shape[1] == 300
    o, lse = ops.attn_fwd(q, k, v, causal=True)
    dq, dk, dv = ops.attn_bwd(q, k, v, o, lse, do, causal=True)
    assert_parity(o, t128("attn_o"), TOL_BF16, "out")
    assert torch.allclose(lse.cpu(), t128("attn_lse"), atol=TOL_LSE, rtol=TOL_LSE)
    for a, n in ((dq, "dq"), (dk, "dk"), (dv, "dv")):
        assert_parity(a, t128(f"attn_{n}"), TOL_BF16, n)
    H, Hkv, D, d, i, L = (int(x) for x in GOLD128["layer_dims"])
    p = {n: t128(f"layer_p_{n}") for n in PARAMS}
    for fused in (True, False):
        layer = _load(OdysseusDecoderLayer(_config(d, H, Hkv, D, i), fused=fused).to(torch.bfloat16), p, dev)
        x = t128("layer_x").to(dev).requires_grad_(True)
        y = layer(x, position_ids=torch.arange(L, device=dev)[None])
        y.backward(t128("layer_dy").to(dev))
        assert rel_err(y, t128("layer_y")) <= TOL_BF16
        got = {"x": x.grad, "ln1": layer.input_layernorm.weight.grad, "w_qkv": layer.self_attn.qkv_proj.weight.grad,
               "w_o": layer.self_attn.o_proj.weight.grad, "ln2": layer.post_attention_layernorm.weight.grad,
               "w_gate_up": layer.mlp.gate_up_proj.weight.grad, "w_down": layer.mlp.down_proj.weight.grad}
        for n, g in got.items():
            assert rel_err(g, t128(f"layer_g_{n}")) <= TOL_BF16, (n, fused)
