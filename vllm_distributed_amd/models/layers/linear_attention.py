"""Linear attention with a decay per head and a recurrent state per request.

Per head ``S_t = decay[h] * S_(t-1) + k_t v_t^T`` and ``o_t = S_t^T q_t``: no softmax, no cache that grows with the
sequence.  What a request carries from token to token is the ``dim x vdim`` matrix ``S`` of every head, in fp32, one
slot per row of the worker's persistent batch (``AttentionMetadata.state_slots``; the model runner allocates the
tensor next to the KV cache and adds a spare slot for the padding rows of captured decode batches).  Nothing is cleared
when a slot changes owner: rows that start at position 0 take the state as zero whatever the slot holds.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch
import torch.nn as nn

from ... import ops
from .attention import get_forward_context


class DecayLinearAttention(nn.Module):
    """Reads ``[q | k | v]`` from the leading columns of a fused projection (``activation``: through SiLU first),
    returns the fp32 heads ``[T, H * vdim]`` side by side."""
    state_dtype = torch.float32

    def __init__(self, num_heads: int, dim: int, vdim: int, decay: Sequence[float], layer_idx: int,
                 activation: bool = True):
        super().__init__()
        if len(decay) != num_heads:
            raise ValueError(f"layer {layer_idx}: {len(decay)} decays for {num_heads} heads")
        self.num_heads, self.dim, self.vdim = num_heads, dim, vdim
        self.layer_idx, self.activation = layer_idx, activation
        # fp32 from the configuration's doubles (the recurrence multiplies by exactly this number every token)
        self.register_buffer("decay", torch.tensor([float(d) for d in decay], dtype=torch.float32), persistent=False)
        self.state: Optional[torch.Tensor] = None

    # ---- per-request state, owned by the model runner
    def state_shape(self, num_slots: int) -> Tuple[int, int, int, int]:
        return (num_slots, self.num_heads, self.dim, self.vdim)

    def state_values_per_slot(self) -> int:
        return self.num_heads * self.dim * self.vdim

    def bind_state(self, state: Optional[torch.Tensor]) -> None:
        self.state = state

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        md = get_forward_context().attn_metadata
        if md is None:                    # memory-profiling pass: no state bound
            return x.new_zeros((x.shape[0], self.num_heads * self.vdim), dtype=torch.float32)
        return ops.decay_linear_attention(x, self.num_heads, self.dim, self.vdim, self.decay, self.state,
                                          md.state_slots, md.query_start_loc, md.seq_lens, self.activation,
                                          md.max_query_len)
