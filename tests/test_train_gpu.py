"""The world-size-1 training step (the reference's train.py loop) on a cut-down model: 2 of the 16 layers,
1024 tokens, 4 steps.  The loss of step 0 is that of a random model (about ln(vocabulary)), every step is
finite, and the weights move."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("mode", ["odysseus", "tpsp"])
def test_training_steps_run(mode, dev, capsys):
    pytest.importorskip("transformers")
    from odysseus_transformer_amd import train
    from odysseus_transformer_amd.utils import globals as g
    print(f"training loop, mode {mode}", flush=True)
    args = train.parse_args(["--use_cfg_init_model", "--parallel_mode", mode, "--num-hidden-layers", "2",
                             "--seq-length", "1024", "--max-train-steps", "4", "--learning-rate", "1e-3"])
    try:
        out = train.main(args)
    finally:
        g._destroy_global_memory_buffer()
    assert out["timed_steps"] == 1 and out["layers"] == 2
    assert all(math.isfinite(l) for l in out["losses"])
    assert abs(out["losses"][0] - math.log(32000)) < 1.5
    text = capsys.readouterr().out
    assert f"{mode} 1K 1 Time taken:" in text and "CUDA memory allocated/reserved" in text


def test_two_training_steps_match_the_oracle_fp32(dev):
    """Two whole fp32 training steps (embedding -> 2 decoder layers -> norm -> lm_head -> fused cross-entropy,
    loss.backward(loss) as the reference's loop does at train.py:214, AdamW) against the oracle's composition
    of decoder_layer_fwd_bwd + rmsnorm + linear + cross_entropy_fwd_bwd + adamw_step in fp64: both losses and
    every weight of the model after the second step, to 1e-4."""
    import types
    from torch import nn
    import odysseus_oracle as oracle
    from conftest import rel_err, randn
    from odysseus_transformer_amd.decoder.odysseus import LlamaRMSNorm, OdysseusDecoderLayer
    from odysseus_transformer_amd.losses.cross_entropy import CrossEntropyLoss
    from odysseus_transformer_amd.optim import AdamW
    from odysseus_transformer_amd.train import NativeLinear

    V, d, H, Hkv, D, i, L, NL, lr = 512, 256, 4, 2, 64, 704, 256, 2, 1e-3
    cfg = types.SimpleNamespace(hidden_size=d, num_attention_heads=H, num_key_value_heads=Hkv, head_dim=D,
                                intermediate_size=i, hidden_act="silu", attention_dropout=0.0, rms_norm_eps=1e-6,
                                rope_theta=10000.0, pretraining_tp=1)
    print("two fp32 training steps vs the oracle", flush=True)

    class Tiny(nn.Module):
        def __init__(self):
            super().__init__()
            self.embed = nn.Embedding(V, d)
            self.layers = nn.ModuleList([OdysseusDecoderLayer(cfg, n) for n in range(NL)])
            self.norm = LlamaRMSNorm(d, 1e-6)
            self.lm_head = NativeLinear(nn.Linear(d, V, bias=False))

        def forward(self, ids, pos):
            h = self.embed(ids)
            for layer in self.layers:
                h = layer(h, position_ids=pos)
            return self.lm_head(self.norm(h))

    model = Tiny().to(torch.float32).to(dev)
    # seeded weights, the same on both sides
    P = {"embed": randn((V, d), 900, std=0.5), "norm": 1.0 + randn((d,), 901, std=0.02), "lm_head": randn((V, d), 902, std=0.05)}
    for n in range(NL):
        P[f"l{n}"] = {"ln1": 1.0 + randn((d,), 910 + 10 * n, std=0.02), "w_qkv": randn(((H + 2 * Hkv) * D, d), 911 + 10 * n, std=0.05),
                      "w_o": randn((d, H * D), 912 + 10 * n, std=0.05), "ln2": 1.0 + randn((d,), 913 + 10 * n, std=0.02),
                      "w_gate_up": randn((2 * i, d), 914 + 10 * n, std=0.05), "w_down": randn((d, i), 915 + 10 * n, std=0.05)}

    def layer_params(layer):
        return {"ln1": layer.input_layernorm.weight, "w_qkv": layer.self_attn.qkv_proj.weight,
                "w_o": layer.self_attn.o_proj.weight, "ln2": layer.post_attention_layernorm.weight,
                "w_gate_up": layer.mlp.gate_up_proj.weight, "w_down": layer.mlp.down_proj.weight}

    with torch.no_grad():
        model.embed.weight.copy_(P["embed"])
        model.norm.weight.copy_(P["norm"])
        model.lm_head.weight.copy_(P["lm_head"])
        for n, layer in enumerate(model.layers):
            for k, t in layer_params(layer).items():
                t.copy_(P[f"l{n}"][k])

    # flat views of the oracle's parameters (fp64) and their AdamW state
    flat = {"embed": P["embed"].double(), "norm": P["norm"].double(), "lm_head": P["lm_head"].double()}
    for n in range(NL):
        for k, t in P[f"l{n}"].items():
            flat[f"l{n}.{k}"] = t.double()
    state = {k: (torch.zeros_like(t), torch.zeros_like(t)) for k, t in flat.items()}

    def oracle_step(ids, labels, step):
        pos = torch.arange(L)[None]
        hs = [flat["embed"][ids]]
        for n in range(NL):
            p = {k: flat[f"l{n}.{k}"] for k in P[f"l{n}"]}
            hs.append(oracle.decoder_layer_fwd(hs[-1], p, H, Hkv, D, position_ids=pos))
        hn = oracle.rmsnorm(hs[-1], flat["norm"])
        logits = oracle.linear_fwd(hn, flat["lm_head"])[0]
        loss, _, _, _ = oracle.cross_entropy_fwd_bwd(logits, labels)
        _, _, _, dlogits = oracle.cross_entropy_fwd_bwd(logits, labels, grad_loss=loss.item())   # loss.backward(loss)
        g = {}
        dhn, g["lm_head"], _ = oracle.linear_bwd(hn, flat["lm_head"], dlogits[None])
        dh, g["norm"] = oracle.rmsnorm_bwd(hs[-1], flat["norm"], dhn)
        for n in reversed(range(NL)):
            p = {k: flat[f"l{n}.{k}"] for k in P[f"l{n}"]}
            _, gl = oracle.decoder_layer_fwd_bwd(hs[n], p, dh, H, Hkv, D, position_ids=pos)
            dh = gl.pop("x")
            for k, t in gl.items():
                g[f"l{n}.{k}"] = t
        g["embed"] = torch.zeros_like(flat["embed"]).index_add_(0, ids[0], dh[0])
        for k in flat:
            m, v = state[k]
            flat[k], m, v = oracle.adamw_step(flat[k], g[k].reshape(flat[k].shape), m, v, step, lr)
            state[k] = (m, v)
        return loss.item()

    optim = AdamW(model.parameters(), lr=lr)
    loss_func = CrossEntropyLoss(inplace_backward=True)
    gen = torch.Generator().manual_seed(5)
    pos = torch.arange(L, device=dev)[None]
    for step in (1, 2):
        batch = torch.randint(V, size=(1, L + 1), generator=gen)
        ids, labels = batch[:, :-1], batch[0, 1:]
        logits = model(ids.to(dev), pos)
        loss = loss_func(logits.reshape(-1, V), labels.to(dev))
        loss.backward(loss)
        optim.step()
        optim.zero_grad()
        want = oracle_step(ids, labels, step)
        print(f"  step {step}: loss {loss.item():.6f}, oracle {want:.6f}", flush=True)
        assert abs(loss.item() - want) <= 1e-4 * max(1.0, abs(want))
    got = {"embed": model.embed.weight, "norm": model.norm.weight, "lm_head": model.lm_head.weight}
    for n, layer in enumerate(model.layers):
        for k, t in layer_params(layer).items():
            got[f"l{n}.{k}"] = t
    # AdamW moves an entry by lr * m / (sqrt(v) + eps): where a gradient is within rounding of zero (|g| ~ eps = 1e-8)
    # the same fp32 rounding error is a different FRACTION of lr, so single entries can be off by a fraction of lr
    # with every kernel exact to 1e-6.  Hence: every weight to 1e-4 in the relative L2 norm, and no entry further off
    # than half a learning-rate step; the second loss above already feels every weight of the first step.
    for k in sorted(flat):
        a, r = got[k].detach().double().cpu(), flat[k]
        l2 = ((a - r).norm() / r.norm()).item()
        worst = (a - r).abs().max().item()
        assert l2 <= 1e-4, f"{k} after two steps: relative L2 error {l2:.3e}"
        assert worst <= 0.5 * lr, f"{k} after two steps: worst entry off by {worst:.3e} (lr = {lr})"


def test_grad_checkpoint_and_profiler_flags(dev, capsys, tmp_path, monkeypatch):
    """--grad-checkpoint (train.py:163-164 of the reference) recomputes every layer in backward: the same losses as
    without it, to the last bit (the kernels are deterministic).  --use_profiler runs the loop inside the reference's
    profiler schedule without disturbing it."""
    pytest.importorskip("transformers")
    from odysseus_transformer_amd import train
    from odysseus_transformer_amd.utils import globals as g
    base = ["--use_cfg_init_model", "--parallel_mode", "odysseus", "--num-hidden-layers", "2", "--seq-length", "1024",
            "--max-train-steps", "4", "--learning-rate", "1e-3"]
    runs = {}
    monkeypatch.chdir(tmp_path)     # the profiler writes ./profile/
    for tag, extra in (("plain", []), ("checkpoint", ["--grad-checkpoint"]), ("profiler", ["--use_profiler"])):
        print(f"training loop with {extra}", flush=True)
        try:
            runs[tag] = train.main(train.parse_args(base + extra))
        finally:
            g._destroy_global_memory_buffer()
    assert runs["checkpoint"]["grad_checkpoint_layers"] == 2 and runs["plain"]["grad_checkpoint_layers"] == 0
    assert runs["checkpoint"]["losses"] == runs["plain"]["losses"]
    assert runs["profiler"]["losses"] == runs["plain"]["losses"]
    assert runs["checkpoint"]["peak_memory_gb"] <= runs["plain"]["peak_memory_gb"]
    assert "gradient checkpointing on for 2 decoder layers" in capsys.readouterr().out
