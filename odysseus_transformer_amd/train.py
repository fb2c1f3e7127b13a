"""World-size-1 training step of the reference's driver (train.py:49-240) on one MI355X.

    python -m odysseus_transformer_amd.train --use_cfg_init_model --parallel_mode odysseus

Same measurement as the reference: `--max-train-steps` steps (10) on random token ids of
`--seq-length` (16384) tokens, the first three untimed, memory printed after model and optimizer
set-up and at every step, `loss.backward(loss)`, AdamW, and one line
"<mode> <L/1024>K <world> Time taken: <s> seconds" at the end (train.py:167-235).  The model is the
16-layer GQA 32/8 configuration of train.py:66-76, randomly initialised (no checkpoint can be
fetched here; `--model` takes a local directory only), patched with
apply_odysseus_attn_patch_llama / apply_tpsp_attn_patch_llama (or, for the ulysses, ring and dp modes,
with the host's attention routed to the HIP flash attention: with one rank their all-to-alls and block
exchanges are the identity), with the loss from the fused cross-entropy kernel.

What differs from the reference and why: one process, one GPU, no FSDP wrapping (its world-size-1
branch skips it too, train.py:118); `--native-host-modules` (default on) also routes the host
model's RMSNorms, lm_head and whatever bias-free projections the patch left in its layers through
the HIP library, so that the step runs on this library's kernels except for the embedding lookup,
the residual adds (and, in the ulysses / ring / dp modes, the rotary embedding and SiLU-multiply)
of the host decoder layer; `--native-optimizer` (default on) runs AdamW as one kernel per tensor
(odysseus_transformer_amd.optim.AdamW) instead of the host framework's element-wise passes.  Switch
either off to keep the host's own modules / optimizer.
"""
from __future__ import annotations

import argparse
import json
import time

import torch
from torch import nn


class NativeLinear(nn.Module):
    """Bias-free nn.Linear on the library's dense products (forward, dgrad, wgrad)."""

    def __init__(self, linear: nn.Linear):
        super().__init__()
        if linear.bias is not None:
            raise NotImplementedError("lm_head with a bias")
        self.weight = linear.weight
        self.in_features, self.out_features = linear.in_features, linear.out_features

    def forward(self, x):
        from .utils.linear_tpsp import _PlainLinearFunc
        return _PlainLinearFunc.apply(x, self.weight)


def use_native_host_modules(model) -> None:
    """Swaps the host model's RMSNorm modules and lm_head for the library's (weights are shared)."""
    from .decoder.odysseus import LlamaRMSNorm

    def native_norm(old):
        new = LlamaRMSNorm(old.weight.shape[0], getattr(old, "variance_epsilon", 1e-6))
        new.weight = old.weight
        return new

    from .decoder.odysseus import OdysseusDecoderLayer
    for layer in model.model.layers:
        if isinstance(layer, OdysseusDecoderLayer):      # already the library's own layer
            continue
        layer.input_layernorm = native_norm(layer.input_layernorm)
        layer.post_attention_layernorm = native_norm(layer.post_attention_layernorm)
        # the host's own projections (the modes that keep its attention / MLP modules: ulysses, ring, dp)
        for parent in (layer.self_attn, layer.mlp):
            for name, child in list(parent.named_children()):
                if type(child) is nn.Linear and child.bias is None:
                    setattr(parent, name, NativeLinear(child))
    model.model.norm = native_norm(model.model.norm)
    model.lm_head = NativeLinear(model.lm_head)


def build_model(args, dev):
    import transformers
    from transformers import LlamaConfig
    if args.use_cfg_init_model:
        cfg = LlamaConfig()
        cfg.hidden_size = 4096
        cfg.intermediate_size = 11008
        cfg.num_attention_heads = 32
        cfg.num_key_value_heads = 8
        cfg.num_hidden_layers = args.num_hidden_layers
        cfg._attn_implementation = "flash_attention_2" if args.declare_flash_attention else "sdpa"
        cfg.rope_theta = args.rope_theta
        if hasattr(cfg, "rope_parameters") and isinstance(cfg.rope_parameters, dict):
            cfg.rope_parameters["rope_theta"] = args.rope_theta
        cfg.max_position_embeddings = max(getattr(cfg, "max_position_embeddings", 0) or 0, args.seq_length)
        cfg.use_cache = False
        with torch.device(dev):                       # initialise on the GPU: 3.1 B parameters take a minute on the host
            model = transformers.LlamaForCausalLM(cfg).to(dtype=torch.bfloat16)
    else:
        import os
        if not os.path.isdir(args.model):
            raise SystemExit(f"--model {args.model!r} is not a local directory and nothing can be downloaded here; "
                             "use --use_cfg_init_model")
        model = transformers.AutoModelForCausalLM.from_pretrained(args.model, torch_dtype=torch.bfloat16)
    return model


def init_prof(use_profiler: bool, out_dir: str = "./profile/"):
    """The reference's profiler context (train.py:28-46): two warm-up and four recorded steps of device activity,
    written as a trace for TensorBoard under ./profile/; a null context without the flag.  Under rocprofv3 leave the
    flag off: every step also opens a named range (torch.profiler.record_function "train_step_<n>") either way."""
    from contextlib import nullcontext
    if not use_profiler:
        return nullcontext()
    return torch.profiler.profile(
        activities=[torch.profiler.ProfilerActivity.CUDA],
        schedule=torch.profiler.schedule(wait=0, warmup=2, active=4, repeat=1),
        on_trace_ready=torch.profiler.tensorboard_trace_handler(out_dir),
        record_shapes=True, with_stack=True)


def enable_grad_checkpoint(model) -> int:
    """--grad-checkpoint (train.py:163-164 calls model.gradient_checkpointing_enable()): every decoder layer's
    activations are dropped after the forward pass and recomputed in backward.  The host model switches its own
    layers on; layers that the patch replaced (OdysseusDecoderLayer) get the same flag.  Returns the number of
    checkpointed layers."""
    from .decoder.odysseus import OdysseusDecoderLayer
    try:
        model.gradient_checkpointing_enable(gradient_checkpointing_kwargs={"use_reentrant": False})
    except Exception as e:   # a host without that switch: the library's own layers below still checkpoint
        print(f"gradient_checkpointing_enable() of the host model failed: {e!r}")
    n = 0
    for layer in model.model.layers:
        if isinstance(layer, OdysseusDecoderLayer):
            layer.gradient_checkpointing = True
            n += 1
        elif getattr(layer, "gradient_checkpointing", False):
            n += 1
    return n


def main(args) -> dict:
    from .decoder.odysseus import apply_odysseus_attn_patch_llama
    from .decoder.tensor_parallel import apply_tpsp_attn_patch_llama
    from .losses.cross_entropy import CrossEntropyLoss
    from .utils.apply_seq_parallel import prepare_attn_inputs
    from .utils.globals import _Arena, _set_global_memory_buffer
    from . import _lib

    assert args.batch_size == 1, "Only support batch size 1"
    if getattr(args, "cpu_offload", False):
        raise NotImplementedError("--cpu-offload is FSDP's parameter offload (train.py:123-157 of the reference); "
                                  "the FSDP wrapping is outside this build")
    rank, world_size = 0, 1
    _lib.load()
    torch.manual_seed(args.seed)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if _Arena.instance is None:
        _set_global_memory_buffer(dev)

    model = build_model(args, dev)
    total_params = sum(p.numel() for p in model.parameters())
    print(f"total parameters {total_params/1e9:.2f}B")
    if args.parallel_mode == "odysseus":
        print(f"use odysseus zero3 {args.use_ody_zero3}")
        with torch.device(dev):
            apply_odysseus_attn_patch_llama(model, use_zero3_linear=args.use_ody_zero3,
                                            fuse_layers=args.fuse_layers and args.use_ody_zero3)
    elif args.parallel_mode == "tpsp":
        with torch.device(dev):
            apply_tpsp_attn_patch_llama(model)
    elif args.parallel_mode == "ulysses":
        from .decoder.ulysses import apply_ulysses_attn_monkey_patch_llama
        apply_ulysses_attn_monkey_patch_llama(model)
    elif args.parallel_mode == "ring":
        from .decoder.ring import apply_zigzag_ring_attn_monkey_patch_llama
        apply_zigzag_ring_attn_monkey_patch_llama(model)
    else:   # dp: the host model as it is; its flash-attention call lands on the HIP kernel (flash_attn is not installed)
        from .decoder.ulysses import install_hip_flash_attention, hip_ulysses_attention_forward
        install_hip_flash_attention(hip_ulysses_attention_forward, model)
    model = model.to(dev)
    from .utils.linear_zero3 import LinearZeRO3
    with torch.no_grad():     # LinearZeRO3 leaves its weight uninitialised, as the reference does: give it finite values
        for m in model.modules():
            if isinstance(m, LinearZeRO3):
                m.weight.normal_(0.0, 0.02)
    if args.native_host_modules:
        use_native_host_modules(model)
    if args.keep_ds_max_gb > 0:
        from . import ops
        ops.set_keep_ds_max_bytes(int(args.keep_ds_max_gb * 1024 ** 3))
    checkpointed = enable_grad_checkpoint(model) if args.grad_checkpoint else 0
    if args.grad_checkpoint:
        print(f"gradient checkpointing on for {checkpointed} decoder layers")
    mem = lambda: (torch.cuda.memory_allocated(dev) / 1024 ** 3, torch.cuda.memory_reserved(dev) / 1024 ** 3)
    print(f"{args.parallel_mode} After init model, CUDA memory allocated: {mem()[0]:.2f} GB, reserved: {mem()[1]:.2f} GB")

    if args.native_optimizer:
        from .optim import AdamW                      # the same update in one pass per tensor
        optim = AdamW(model.parameters(), lr=args.learning_rate)
    else:
        optim = torch.optim.AdamW(model.parameters(), lr=args.learning_rate)
    model.train()
    loss_func = CrossEntropyLoss(inplace_backward=True)
    warmup_num_iterations = 2
    elapse, step_times, losses = 0.0, [], []
    print(f"{args.parallel_mode} After init optim, CUDA memory allocated: {mem()[0]:.2f} GB, reserved: {mem()[1]:.2f} GB")

    gen = torch.Generator().manual_seed(args.seed)
    vocab_size = model.config.vocab_size
    with init_prof(args.use_profiler) as prof:
        for step in range(args.max_train_steps):
            if step > warmup_num_iterations:
                start_time = time.time()
            with torch.profiler.record_function(f"train_step_{step}"):
                batch = torch.randint(vocab_size, size=(1, args.seq_length + 1), generator=gen)
                input_ids, target_ids = batch[..., :-1], batch[..., 1:]
                position_ids = torch.arange(args.seq_length).unsqueeze(0).expand(input_ids.shape[0], -1)
                prepared = prepare_attn_inputs(args.parallel_mode, input_ids, position_ids, target_ids, rank, world_size, dev)
                logits = model(prepared["local_input_ids"], position_ids=prepared["local_position_ids"], use_cache=False).logits
                loss = loss_func(logits.reshape(-1, logits.shape[-1]), prepared["local_target_ids"].reshape(-1))
                print(f"step {step} CUDA memory allocated/reserved: {mem()[0]:.2f}/{mem()[1]:.2f} GB")
                losses.append(loss.item())
                print(f"loss {losses[-1]}", flush=True)
                loss.backward(loss)
                optim.step()
                optim.zero_grad()
            if step >= warmup_num_iterations:
                # the reference starts and stops its clock without one, so that a timed step pays for the queued tail of
                # the step before it; here the seven timed steps are seven whole steps
                torch.cuda.synchronize()
            if step > warmup_num_iterations:
                step_times.append(time.time() - start_time)
                elapse += step_times[-1]
            if args.use_profiler:
                prof.step()
    print(f"{args.parallel_mode} {args.seq_length//1024}K {world_size} Time taken: {elapse:.2f} seconds")
    out = {"parallel_mode": args.parallel_mode, "seq_length": args.seq_length, "layers": model.config.num_hidden_layers,
           "parameters_b": round(total_params / 1e9, 3), "timed_steps": len(step_times), "time_taken_s": round(elapse, 3),
           "step_ms": [round(1e3 * t, 1) for t in step_times], "tokens_per_s": round(args.seq_length * len(step_times) /
                                                                                      max(elapse, 1e-9), 1),
           "peak_memory_gb": round(torch.cuda.max_memory_allocated(dev) / 1024 ** 3, 2), "losses": [round(l, 4) for l in losses],
           "native_host_modules": bool(args.native_host_modules), "native_optimizer": bool(args.native_optimizer),
           "fuse_layers": bool(args.fuse_layers and args.parallel_mode == "odysseus"),
           "grad_checkpoint_layers": checkpointed, "keep_ds_max_gb": args.keep_ds_max_gb}
    print(json.dumps(out))
    return out


def parse_args(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--batch-size", type=int, default=1)
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--max-train-steps", type=int, default=10)
    ap.add_argument("--learning-rate", type=float, default=2e-5)
    ap.add_argument("--rope-theta", type=float, default=100000)
    ap.add_argument("--model", type=str, default="meta-llama/Llama-2-7b-hf")
    ap.add_argument("--seq-length", type=int, default=16384)
    ap.add_argument("--grad-checkpoint", action="store_true", default=False,
                    help="drop every decoder layer's activations after the forward pass and recompute them in backward")
    ap.add_argument("--cpu-offload", action="store_true", default=False,
                    help="accepted for command-line compatibility (train.py:252 of the reference): FSDP's parameter "
                         "offload to the host is part of the FSDP wrapping, which is outside this build; refused")
    ap.add_argument("--use_zero2", action="store_true", default=False,
                    help="accepted for command-line compatibility (train.py:254): FSDP's SHARD_GRAD_OP strategy; with one "
                         "rank there is nothing to shard, so it changes nothing here")
    ap.add_argument("--use_ody_zero3", action="store_true", default=True)
    ap.add_argument("--use_profiler", action="store_true", default=False,
                    help="torch.profiler over steps 2-5 (two warm-up, four recorded), trace under ./profile/")
    ap.add_argument("--use_cfg_init_model", action="store_true", default=False)
    ap.add_argument("--parallel_mode", type=str, choices=["odysseus", "ulysses", "dp", "tpsp", "ring"], default="odysseus")
    ap.add_argument("--num-hidden-layers", type=int, default=16, help="16 in the reference's configuration (train.py:71)")
    ap.add_argument("--native-host-modules", action=argparse.BooleanOptionalAction, default=True)
    ap.add_argument("--fuse-layers", action=argparse.BooleanOptionalAction, default=True,
                    help="odysseus mode: swap whole decoder layers (residual adds inside the projections' epilogues) "
                         "instead of the attention and MLP modules only, as the reference's patch does")
    ap.add_argument("--native-optimizer", action=argparse.BooleanOptionalAction, default=True,
                    help="AdamW as one HIP kernel per tensor instead of torch.optim.AdamW's element-wise passes")
    ap.add_argument("--keep-ds-max-gb", type=float, default=0.0,
                    help="memory the attention backward may spend on kept dS (about Hq * L * L bytes per layer call, one "
                         "buffer shared by all layers: 8 GiB at 32 heads x 16384 tokens) for a few percent of speed; "
                         "0 = the recomputing kernels")
    ap.add_argument("--declare-flash-attention", action=argparse.BooleanOptionalAction, default=False,
                    help="set config._attn_implementation before the model is built (needs flash_attn importable); "
                         "the patchers set it afterwards either way")
    return ap.parse_args(argv)


if __name__ == "__main__":
    main(parse_args())
