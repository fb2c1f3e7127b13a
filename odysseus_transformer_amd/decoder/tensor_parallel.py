"""Tensor-parallel + sequence-parallel SwiGLU MLP and the TP-SP module patcher
(decoder/tensor_parallel.py of the reference) on the gfx950 HIP library.

One rank's share: the gate and up projections are column-split (this rank's rows of W1 and W3,
packed as [W1 rows ; W3 rows] in `w1w3`), the down projection is row-split (this rank's columns
of W2) and its partial sums are reduce-scattered along the sequence.  At world_size = 1 the shards
are the full weights and the collectives are the identity; larger groups raise at the collective.
"""
from __future__ import annotations

import torch
from torch import nn

from .. import ops
from ..utils.allgather import allgather_bsz1
from ..utils.linear_tpsp import ColumnParallelLinear, ColumnParallelLinearAG, RowParallelLinearRS
from .odysseus import LlamaFlashAttention2TPSP, _host_builds_no_mask, _host_layer_unpacks_two


class LlamaMLPTPSP(nn.Module):
    """down(silu(gate(x)) * up(x)) with Megatron-style sharding (decoder/tensor_parallel.py:14-85).

    Args (as the reference):
        pack_weight: one packed projection `w1w3` (gate rows first, then up rows) or two (`w1`, `w3`).
        sequence_parallel: the packed projection gathers the sequence itself.
        keep_master_weight_for_test: keep the unsplit weight of each sharded linear.
    """

    def __init__(self, config, pack_weight: bool = True, sequence_parallel=True, keep_master_weight_for_test=False):
        super().__init__()
        self.config = config
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.intermediate_size
        act = getattr(config, "hidden_act", "silu")
        if act != "silu":
            raise NotImplementedError(f"hidden_act={act!r}: only the SiLU gate of Llama is implemented")
        self.act_fn = torch.nn.functional.silu  # for introspection; the fused kernel applies it
        use_bias = False
        self.pack_weight = pack_weight
        self.sequence_parallel = sequence_parallel
        kw = dict(bias=use_bias, gather_output=False, keep_master_weight_for_test=keep_master_weight_for_test)
        if pack_weight:
            cls = ColumnParallelLinearAG if sequence_parallel else ColumnParallelLinear
            self.w1w3 = cls(self.hidden_size, self.intermediate_size * 2, **kw)
        else:
            self.w1 = ColumnParallelLinear(self.hidden_size, self.intermediate_size, **kw)
            self.w3 = ColumnParallelLinear(self.hidden_size, self.intermediate_size, **kw)
        self.w2 = RowParallelLinearRS(self.intermediate_size, self.hidden_size, bias=use_bias, input_is_parallel=True,
                                      keep_master_weight_for_test=keep_master_weight_for_test)

    def forward(self, x):
        assert getattr(self.config, "pretraining_tp", 1) <= 1, "Pretraining TP is not supported for LlamaMLP"
        if self.pack_weight:
            if not self.sequence_parallel:
                x = allgather_bsz1(x)
            return self.w2(ops.swiglu(self.w1w3(x)))
        x = allgather_bsz1(x)
        # the fused SwiGLU kernel reads [gate | up] side by side: write both projections into one buffer
        return self.w2(ops.swiglu(torch.cat((self.w1(x), self.w3(x)), dim=-1)))


def apply_tpsp_attn_patch_llama(model):
    """Swaps every layer's attention and MLP for the TP-SP modules (decoder/tensor_parallel.py:88-97).
    As in the reference the new modules are freshly initialised."""
    _host_builds_no_mask(model)
    for i in range(model.config.num_hidden_layers):
        layer = model.model.layers[i]
        new_attn = LlamaFlashAttention2TPSP(model.config, i).to(model.dtype)
        if _host_layer_unpacks_two(layer):
            new_attn.return_arity = 2
        layer.self_attn = new_attn
        layer.mlp = LlamaMLPTPSP(model.config).to(model.dtype)
    print("Applied TP-SP patch for LlamaFlashAttn")
