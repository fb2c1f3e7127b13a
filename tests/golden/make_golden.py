#!/usr/bin/env python3
"""Writes tests/golden/llama_layer_small.npz and tests/golden/llama_d128.npz: inputs, parameters, output and every gradient
of ONE Llama decoder layer (RMSNorm -> packed QKV -> RoPE -> causal GQA attention -> O ->
residual -> RMSNorm -> SwiGLU MLP -> residual).

The numbers come from the INSTALLED transformers' LlamaDecoderLayer (eager attention) run in
fp64 with torch.autograd -- a library implementation independent of the CPU oracle -- plus
torch's scaled_dot_product_attention for a stand-alone attention case with its log-sum-exp
from torch.logsumexp.  The reference repository ships no vectors for this path; these stand
in for them and pin the oracle (CPU test) and the HIP path (GPU test) to fixed data.

llama_layer_small.npz holds head_dim 64 (fp32 kernels); llama_d128.npz holds head_dim 128 with
grouped-query attention and lengths that span more than one 256-query block with a ragged last
tile (300 and 260 tokens), inputs rounded to bfloat16 (stored as their 16-bit patterns) so that the
bf16 MFMA kernels behind every benchmark number run on exactly the data the fp64 results belong to.

Run from the repository root:  python tests/golden/make_golden.py
"""
from pathlib import Path

import numpy as np
import torch
import torch.nn.functional as F
from transformers.models.llama import modeling_llama as ml

HERE = Path(__file__).resolve().parent
F64 = torch.float64

# head_dim 64 so that the same vectors run through the HIP kernels
H, HKV, D, DM, I, L = 2, 1, 64, 64, 96, 40


def randn(shape, seed, std=1.0, bf16_exact=False):
    g = torch.Generator(device="cpu").manual_seed(seed)
    t = torch.randn(shape, generator=g, dtype=torch.float32) * std
    if bf16_exact:
        t = t.bfloat16().float()
    return t.to(F64)


def layer_case(H=H, HKV=HKV, D=D, DM=DM, I=I, L=L, bf=False, seed=0):
    r = lambda shape, k, std=1.0: randn(shape, seed + k, std, bf)
    one = lambda k: (1 + randn((DM,), seed + k, 0.1)).float().bfloat16().to(F64) if bf else 1 + randn((DM,), seed + k, 0.1)
    p = {"ln1": one(1), "w_qkv": r(((H + 2 * HKV) * D, DM), 2, 0.1),
         "w_o": r((DM, H * D), 3, 0.1), "ln2": one(4),
         "w_gate_up": r((2 * I, DM), 5, 0.1), "w_down": r((DM, I), 6, 0.1)}
    x, dy = r((1, L, DM), 7), r((1, L, DM), 8)
    cfg = ml.LlamaConfig(hidden_size=DM, intermediate_size=I, num_attention_heads=H, num_key_value_heads=HKV,
                         head_dim=D, rms_norm_eps=1e-6, attention_bias=False, mlp_bias=False, rope_theta=10000.0)
    cfg._attn_implementation = "eager"
    layer = ml.LlamaDecoderLayer(cfg, 0).to(F64)
    rot = ml.LlamaRotaryEmbedding(cfg)
    with torch.no_grad():
        layer.input_layernorm.weight.copy_(p["ln1"])
        layer.post_attention_layernorm.weight.copy_(p["ln2"])
        layer.self_attn.q_proj.weight.copy_(p["w_qkv"][:H * D])
        layer.self_attn.k_proj.weight.copy_(p["w_qkv"][H * D:(H + HKV) * D])
        layer.self_attn.v_proj.weight.copy_(p["w_qkv"][(H + HKV) * D:])
        layer.self_attn.o_proj.weight.copy_(p["w_o"])
        layer.mlp.gate_proj.weight.copy_(p["w_gate_up"][:I])
        layer.mlp.up_proj.weight.copy_(p["w_gate_up"][I:])
        layer.mlp.down_proj.weight.copy_(p["w_down"])
    pos = torch.arange(L)[None]
    cos, sin = rot(x, pos)
    mask = torch.full((L, L), float("-inf"), dtype=F64).triu(1)[None, None]
    xl = x.clone().requires_grad_()
    out = layer(xl, attention_mask=mask, position_ids=pos, position_embeddings=(cos.to(F64), sin.to(F64)))
    out = out[0] if isinstance(out, tuple) else out
    out.backward(dy)
    a = layer.self_attn
    g = {"x": xl.grad, "ln1": layer.input_layernorm.weight.grad, "ln2": layer.post_attention_layernorm.weight.grad,
         "w_qkv": torch.cat((a.q_proj.weight.grad, a.k_proj.weight.grad, a.v_proj.weight.grad), 0),
         "w_o": a.o_proj.weight.grad,
         "w_gate_up": torch.cat((layer.mlp.gate_proj.weight.grad, layer.mlp.up_proj.weight.grad), 0),
         "w_down": layer.mlp.down_proj.weight.grad}
    d = {"layer_dims": np.array([H, HKV, D, DM, I, L]), "layer_x": x, "layer_dy": dy, "layer_y": out.detach()}
    d.update({f"layer_p_{k}": v for k, v in p.items()})
    d.update({f"layer_g_{k}": v for k, v in g.items()})
    return d


def attention_case(Lq=70, Hq=4, Hkv=2, D=D, bf=False, seed=0):
    """(B, L, H, D) = (1, 70, 4, 64) queries against 2 KV heads, causal: SDPA + autograd in fp64."""
    r = lambda shape, k: randn(shape, seed + k, 1.0, bf)
    q, do = r((1, Lq, Hq, D), 11).requires_grad_(), r((1, Lq, Hq, D), 12)
    k, v = r((1, Lq, Hkv, D), 13).requires_grad_(), r((1, Lq, Hkv, D), 14).requires_grad_()
    o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True,
                                       enable_gqa=True).transpose(1, 2)
    o.backward(do)
    kk = k.detach().repeat_interleave(Hq // Hkv, 2)
    s = torch.einsum("blhd,bmhd->bhlm", q.detach(), kk) / D ** 0.5
    s = s.masked_fill(torch.ones(Lq, Lq, dtype=torch.bool).triu(1), float("-inf"))
    return {"attn_q": q.detach(), "attn_k": k.detach(), "attn_v": v.detach(), "attn_do": do, "attn_o": o.detach(),
            "attn_lse": torch.logsumexp(s, -1), "attn_dq": q.grad, "attn_dk": k.grad, "attn_dv": v.grad}


def main():
    torch.manual_seed(0)
    d = {}
    d.update(layer_case())
    d.update(attention_case())
    arrays = {k: (v if isinstance(v, np.ndarray) else v.detach().to(torch.float32).numpy()) for k, v in d.items()}
    np.savez_compressed(HERE / "llama_layer_small.npz", **arrays)
    print("wrote", HERE / "llama_layer_small.npz", sum(a.nbytes for a in arrays.values()), "bytes of arrays")
    # head_dim 128, GQA 2:1, ragged lengths beyond one 256-query block; inputs are bf16-exact
    d = {}
    d.update(layer_case(H=2, HKV=1, D=128, DM=128, I=192, L=260, bf=True, seed=100))
    d.update(attention_case(Lq=300, Hq=2, Hkv=1, D=128, bf=True, seed=100))
    inputs = {"layer_x", "layer_dy", "attn_q", "attn_k", "attn_v", "attn_do"} | {k for k in d if k.startswith("layer_p_")}
    arrays = {}
    for k, v in d.items():
        if isinstance(v, np.ndarray):
            arrays[k] = v
        elif k in inputs:     # exact in bfloat16: keep the 16-bit patterns
            arrays[k + "_bf16bits"] = v.detach().to(torch.bfloat16).view(torch.int16).numpy()
        else:
            arrays[k] = v.detach().to(torch.float32).numpy()
    np.savez_compressed(HERE / "llama_d128.npz", **arrays)
    print("wrote", HERE / "llama_d128.npz", sum(a.nbytes for a in arrays.values()), "bytes of arrays")


if __name__ == "__main__":
    main()
