"""Zigzag ring attention of the reference (decoder/ring.py) on the gfx950 HIP library: what ONE rank computes.

The reference routes HF's flash-attention call to ring_flash_attn's zigzag_ring_flash_attn_func
(decoder/ring.py:8,30-37) and feeds every rank chunks r and 2N-1-r of the sequence
(utils/apply_seq_parallel.py:93-129).  The exchange of K/V blocks between ranks is a collective and is not
built; the arithmetic of a rank is:

  * zigzag_ring_rank_attn(q, k_blocks, v_blocks, rank, world_size): the rank's N steps with the blocks it
    would receive passed in (block s = local K/V of rank (r - s) mod N), forward and backward;
  * zigzag_ring_flash_attn_func(q, k, v, ...): the reference's call signature; with a world of one rank the
    two local chunks are the whole sequence and the ring has the single causal step.

apply_zigzag_ring_attn_monkey_patch_llama() routes the host model's attention to it, as the reference's patch
does.  The reference also replaces LlamaDecoderLayer.forward with a copy of the host's own
(decoder/ring.py:40-95); that changes nothing and has no counterpart here.
"""
from __future__ import annotations

from typing import Optional

from .. import ops, parallel_state
from .ulysses import install_hip_flash_attention

zigzag_ring_rank_attn = ops.zigzag_ring_rank_attn


def zigzag_ring_flash_attn_func(q, k, v, dropout_p: float = 0.0, softmax_scale: Optional[float] = None,
                                causal: bool = False, return_lse: bool = False):
    """q (B, 2c, Hq, D), k / v (B, 2c, Hkv, D): this rank's two chunks.  World size 1 only (beyond it the K/V
    blocks travel between ranks; use zigzag_ring_rank_attn with the blocks in hand)."""
    if parallel_state.get_model_parallel_world_size() != 1:
        raise NotImplementedError("the exchange of K/V blocks between ranks is not part of this build; "
                                  "zigzag_ring_rank_attn computes one rank's steps from the blocks it is given")
    if not causal:
        raise NotImplementedError("the zigzag split only makes sense for causal attention")
    return ops.flash_attn_func(q, k, v, dropout_p, softmax_scale, causal=True, return_lse=return_lse)


def hip_zigzag_ring_attention_forward(module, query, key, value, attention_mask, dropout=0.0, scaling=None, **kwargs):
    """HF attention-interface entry: (B, H, L, D) tensors in, (B, L, H, D) out (decoder/ring.py:10-37)."""
    assert attention_mask is None, "padded batches are not supported (decoder/ring.py:27)"
    assert getattr(module, "is_causal", True) is True
    assert kwargs.get("sliding_window") is None, "sliding windows are not supported (decoder/ring.py:29)"
    out = zigzag_ring_flash_attn_func(query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2), dropout,
                                      scaling, causal=True)
    return out, None


def apply_zigzag_ring_attn_monkey_patch_llama(model=None) -> None:
    """decoder/ring.py:98-104.  Pass the model so that its config asks for the flash-attention entry."""
    install_hip_flash_attention(hip_zigzag_ring_attention_forward, model)


def apply_zigzag_ring_attn_monkey_patch_mistral(model=None) -> None:
    """decoder/ring.py:107-113: the same routing for a Mistral host.  The reference assigns to
    MistralFlashAttention2._flash_attention_forward; the installed transformers reaches every model family's
    flash-attention call through one registry, so the entry is the one the Llama patch installs.  A Mistral
    config with a sliding window is refused at the call, as the reference does (decoder/ring.py:29)."""
    install_hip_flash_attention(hip_zigzag_ring_attention_forward, model)


# the names the reference's train.py imports (train.py:23)
apply_zigzag_ring_attn_patch_llama = apply_zigzag_ring_attn_monkey_patch_llama
apply_zigzag_ring_attn_patch_mistral = apply_zigzag_ring_attn_monkey_patch_mistral
