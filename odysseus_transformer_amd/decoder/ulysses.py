"""DeepSpeed-Ulysses attention of the reference (decoder/ulysses.py) on the gfx950 HIP library: what ONE rank
computes.

Ulysses turns sequence shards into head shards with an all-to-all before attention and back after it
(yunchang's UlyssesAttention, decoder/ulysses.py:8-10,36-43); between the two a rank runs plain causal flash
attention over the full sequence on its heads -- the same kernel call as the Odysseus module's.  The
all-to-alls are collectives and are not built: with a world of one rank they are the identity and the call
is the flash attention itself.  apply_ulysses_attn_monkey_patch_llama() routes the host model's attention
there, as the reference's patch does (decoder/ulysses.py:108-114).
"""
from __future__ import annotations

from .. import ops, parallel_state


def install_hip_flash_attention(fn, model=None) -> None:
    """Makes `fn` the host's "flash_attention_2" attention entry (what the reference does by assigning to
    LlamaFlashAttention2._flash_attention_forward) and, given a model, declares that implementation in its
    config so that the host builds no dense mask."""
    from transformers import AttentionInterface
    AttentionInterface.register("flash_attention_2", fn)
    if model is not None:
        model.config._attn_implementation = "flash_attention_2"


def ulysses_attn(q, k, v, dropout_p: float = 0.0, softmax_scale=None, causal: bool = False):
    """(B, L/N, H, D) per rank in the reference; with one rank (B, L, H, D) straight into the kernel."""
    if parallel_state.get_model_parallel_world_size() != 1:
        raise NotImplementedError("the all-to-all between sequence and head shards is not part of this build")
    return ops.flash_attn_func(q, k, v, dropout_p, softmax_scale, causal=causal)


def hip_ulysses_attention_forward(module, query, key, value, attention_mask, dropout=0.0, scaling=None, **kwargs):
    """HF attention-interface entry: (B, H, L, D) tensors in, (B, L, H, D) out (decoder/ulysses.py:18-45)."""
    assert attention_mask is None, "padded batches are not supported (decoder/ulysses.py:33)"
    assert getattr(module, "is_causal", True) is True
    assert kwargs.get("sliding_window") is None, "sliding windows are not supported (decoder/ulysses.py:35)"
    out = ulysses_attn(query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2), dropout, scaling, causal=True)
    return out, None


def apply_ulysses_attn_monkey_patch_llama(model=None) -> None:
    """decoder/ulysses.py:108-114.  Pass the model so that its config asks for the flash-attention entry."""
    install_hip_flash_attention(hip_ulysses_attention_forward, model)
